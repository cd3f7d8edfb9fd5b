"""Kikelorn on the GPU: every mechanism's kernel alone against the plain functions of oracle/kikelorn.py, then the engine
(scheduler commit, pages, state slots, run_portions) against the oracle run on each request's whole token list."""

import pytest
import torch

from kikelorn_cases import (Engine, aligned_config, engine_config, mixed_config, odd_config, plain_config,
                            random_checkpoint, random_config, row_error, row_errors)
from oracle import kikelorn as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64
F32_TOL, BF16_TOL = 2e-4, 6e-2          # engine logits against the float64 oracle (row_error)
SAME_TOL = 2e-5                         # fp32 engine against itself under another schedule


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


def _round(t, dtype):
    return t.to(dtype).float()


PIECES = [[40], [1] * 40, [2, 2, 33, 1, 2], [17, 16, 7], [39, 1]]


# ------------------------------------------------------------------------------------------------ post-norm residual
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [100, 96, 1030])
@pytest.mark.parametrize("gated", [True, False])
def test_gated_postnorm_add(dtype, n, gated):
    from byox_vllm_amd import kernels
    g = torch.Generator().manual_seed(n)
    x, y = torch.randn(9, n, generator=g), torch.randn(9, n + 3, generator=g) * 4
    logits, bias = torch.randn(9, n + 5, generator=g) * 2, _round(torch.randn(n, generator=g), dtype)
    w = _round(1 + 0.3 * torch.randn(n, generator=g), dtype)
    xd = x.to(DEV)
    yb = _round(torch.randn(n, generator=g), dtype) if n != 96 else None       # a bias its product left to be added here
    out = kernels.gated_postnorm_add(xd, y.to(DEV)[:, 3:], w.to(DEV).to(dtype), 1e-5, 0.7,
                                     gate=logits.to(DEV)[:, 5:] if gated else None,
                                     gate_bias=bias.to(DEV).to(dtype) if gated else None, out_dtype=dtype,
                                     y_bias=yb.to(DEV).to(dtype) if yb is not None else None)
    gy = y[:, 3:].double() + (yb.double() if yb is not None else 0.0)
    gy = gy * (torch.sigmoid(logits[:, 5:].double() + bias.double()) if gated else 1.0)
    want = x.double() + 0.7 * O.rms(gy, 1e-5) * w.double()
    _close(xd, want, 1e-6)                                         # the residual itself stays fp32
    assert torch.equal(out.cpu(), xd.cpu().to(dtype))
    # nothing pending: a copy in the model dtype, the residual untouched
    before = xd.clone()
    copy = kernels.gated_postnorm_add(xd, None, None, 0.0, 0.0, out_dtype=dtype)
    assert torch.equal(xd, before) and torch.equal(copy, before.to(dtype))


def test_postnorm_eps_sits_inside_the_root():
    """A result of all zeros must add nothing (and no NaN); a tiny one is damped by eps, not blown up to norm one."""
    from byox_vllm_amd import kernels
    x = torch.ones(2, 64, device=DEV)
    y = torch.zeros(2, 64, device=DEV)
    y[1] = 1e-4
    kernels.gated_postnorm_add(x, y, torch.ones(64, device=DEV), 1e-2, 1.0)
    want = 1.0 + 1e-4 / (1e-8 + 1e-2) ** 0.5
    assert torch.equal(x[0].cpu(), torch.ones(64)) and abs(float(x[1, 0]) - want) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,taps", [(100, 3), (96, 1), (2048, 4), (1028, 2), (4096, 5)])
def test_postnorm_launch_runs_the_next_input_convolution_for_single_tokens(dtype, n, taps):
    """Three requests decode side by side, one joins later in a slot another has left, one sits a step out: the fused
    launch must give the residual of the plain launch and x + conv(x) of the whole sequences."""
    from byox_vllm_amd import kernels
    g = torch.Generator().manual_seed(n + taps)
    lens = {"a": 9, "b": 4, "c": 7, "d": 5}
    ys = {k: torch.randn(v, n, generator=g) * 3 for k, v in lens.items()}
    w = _round(1 + 0.3 * torch.randn(n, generator=g), dtype)
    cw = _round(torch.randn(n, taps, generator=g) * 0.5, dtype)
    # the residual of a request: x_t = x0_t + 0.5 * rms(y_t) * w, rows independent of each other
    x0 = {k: torch.randn(v, n, generator=g) for k, v in lens.items()}
    xs = {k: x0[k].double() + 0.5 * O.rms(ys[k].double(), 1e-5) * w.double() for k in lens}
    want = {k: xs[k] + O.causal_conv(xs[k], cw.double()) for k in lens}
    state = torch.full((4, taps - 1, n), float("nan"), device=DEV)
    at = {k: 0 for k in lens}
    slot = {"a": 0, "b": 2, "c": 1}
    steps = [["a", "b", "c"], ["a", "b"], ["a", "b", "c"], ["b", "c", "a"], ["a", "c", "d"], ["d", "a", "c"], ["c", "d", "a"],
             ["a", "d", "c"], ["d", "a", "c"], ["a"]]
    for names in steps:
        if "d" in names and "d" not in slot:
            slot["d"] = slot["b"]                     # b is over: its slot is used again
        names = [k for k in names if at[k] < lens[k]]
        if not names:
            continue
        x = torch.stack([x0[k][at[k]] for k in names]).to(DEV)
        y = torch.stack([ys[k][at[k]] for k in names]).to(DEV)
        rows, h = kernels.gated_postnorm_add(x, y, w.to(DEV).to(dtype), 1e-5, 0.5, out_dtype=dtype,
                                             conv=(cw.to(DEV).to(dtype), state, _i32([slot[k] for k in names]),
                                                   _i32([at[k] for k in names])))
        for i, k in enumerate(names):
            _close(x[i], xs[k][at[k]], 1e-6)
            _close(h[i].float(), want[k][at[k]], 2e-6 if dtype == torch.float32 else 8e-3)
            at[k] += 1
        assert torch.equal(rows, x.to(dtype))
    assert at == lens and torch.isnan(state[3]).all()


# ------------------------------------------------------------------------------------------------ input convolution
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
@pytest.mark.parametrize("pieces", PIECES)
@pytest.mark.parametrize("C", [70, 72])
def test_input_convolution_in_pieces(dtype, taps, pieces, C):
    """x + conv(x) over one request cut into pieces down to one token, from a slot that held something else; channel
    counts that do and do not split into groups of four."""
    from byox_vllm_amd import kernels
    T = 40
    g = torch.Generator().manual_seed(taps)
    x = torch.randn(T, C + 4, generator=g)
    w = _round(torch.randn(C, taps, generator=g) * 0.5, dtype)
    state = torch.full((3, taps - 1, C), float("nan"), device=DEV)
    xd, wd, outs = x.to(DEV), w.to(DEV).to(dtype), []
    for a, n, cu, past, slots, seq_of in _steps(pieces, slot=2):
        outs.append(kernels.causal_conv(xd[a:a + n, 4:], wd, None, state, cu, past, slots, seq_of, act=2, want_f32=True,
                                        want_t=True))
    want = x[:, 4:].double() + O.causal_conv(x[:, 4:].double(), w.double())
    _close(torch.cat([o[0] for o in outs]), want, 1e-6)
    assert torch.equal(torch.cat([o[1] for o in outs]), torch.cat([o[0] for o in outs]).to(dtype))
    assert torch.isnan(state[:2]).all() and not torch.isnan(state[2]).any()


@pytest.mark.parametrize("C", [33, 64])
def test_input_convolution_keeps_requests_apart(C):
    """Two requests in one launch, the second continuing from its slot: no tap reaches into the neighbour's rows."""
    from byox_vllm_amd import kernels
    taps = 4
    g = torch.Generator().manual_seed(0)
    xa, xb = torch.randn(6, C, generator=g), torch.randn(9, C, generator=g)
    w = torch.randn(C, taps, generator=g)
    state = torch.zeros(2, taps - 1, C, device=DEV)
    wd = w.to(DEV)
    first = kernels.causal_conv(xb[:4].to(DEV), wd, None, state, _i32([0, 4]), _i32([0]), _i32([1]), _i32([0] * 4), act=2)[0]
    both = kernels.causal_conv(torch.cat([xa, xb[4:]]).to(DEV), wd, None, state, _i32([0, 6, 11]), _i32([0, 4]), _i32([0, 1]),
                               _i32([0] * 6 + [1] * 5), act=2)[0]
    _close(both[:6], xa.double() + O.causal_conv(xa.double(), w.double()), 1e-6)
    _close(torch.cat([first, both[6:]]), xb.double() + O.causal_conv(xb.double(), w.double()), 1e-6)


# ------------------------------------------------------------------------------------------------ minGRU
def _mingru_plain(proj, offs, C, zb, ub):
    p = proj.double()
    z = torch.sigmoid(p[:, offs[0]:offs[0] + C] + zb.double())
    u = p[:, offs[1]:offs[1] + C] + ub.double()
    return O.min_gru(z, u) * O.silu(p[:, offs[2]:offs[2] + C])


def _mingru_run(proj, offs, C, zb, ub, pieces, state, slot, dtype=torch.float32, past=0):
    from byox_vllm_amd import kernels
    pd, outs = proj.to(DEV), []
    for a, n, cu, pl, slots, _ in _steps(pieces, slot, past):
        out = torch.zeros(n, C + 1, dtype=dtype, device=DEV)
        kernels.mingru_scan(pd[a:a + n], offs, zb.to(DEV).to(dtype), ub.to(DEV).to(dtype), state, cu, pl, slots, C, out[:, 1:])
        assert float(out[:, 0].float().abs().max()) == 0.0
        outs.append(out[:, 1:])
    return torch.cat(outs).float()


@pytest.mark.parametrize("C", [70, 64, 200, 1])
@pytest.mark.parametrize("pieces", PIECES + [[16, 16, 8], [3, 37]])
def test_mingru_in_pieces(C, pieces):
    g = torch.Generator().manual_seed(C)
    proj = torch.randn(40, 3 * C + 4, generator=g) * 2
    offs = (4 + C, 4, 4 + 2 * C)                                   # candidates first, then the gate, then the output gate
    zb, ub = torch.randn(C, generator=g), torch.randn(C, generator=g)
    state = torch.full((3, C), float("nan"), device=DEV)
    got = _mingru_run(proj, offs, C, zb, ub, pieces, state, slot=1)
    _close(got, _mingru_plain(proj, offs, C, zb, ub), 2e-6)
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all() and not torch.isnan(state[1]).any()


def test_mingru_candidate_has_two_branches():
    """u >= 0 gives u + 1/2 (also at zero itself), u < 0 the sigmoid; with the gate wide open the state IS the candidate."""
    C = 5
    proj = torch.zeros(1, 3 * C)
    proj[0, :C] = 40.0
    proj[0, C:2 * C] = torch.tensor([0.0, -0.0, 3.0, -3.0, -1e-6])
    proj[0, 2 * C:] = 30.0                                         # silu(30) = 30
    state = torch.zeros(1, C, device=DEV)
    got = _mingru_run(proj, (0, C, 2 * C), C, torch.zeros(C), torch.zeros(C), [1], state, 0) / 30.0
    want = torch.tensor([0.5, 0.5, 3.5, float(torch.sigmoid(torch.tensor(-3.0))), 0.5])
    assert float((got[0].cpu() - want).abs().max()) < 1e-5


@pytest.mark.parametrize("pieces", [[400], [200, 1, 199], [3] + [1] * 397, [5, 395]])
def test_mingru_holds_a_value_for_hundreds_of_tokens(pieces):
    """Channel 0 opens its gate at token 3 only and must still show that candidate at token 399; channel 1 never closes
    and follows the current token; channel 2 never opens and stays at zero."""
    C, T = 3, 400
    g = torch.Generator().manual_seed(1)
    proj = torch.zeros(T, 3 * C)
    proj[:, C:2 * C] = torch.randn(T, C, generator=g)
    proj[:, 0], proj[3, 0] = -40.0, 40.0
    proj[:, 1], proj[:, 2] = 40.0, -40.0
    proj[:, 2 * C:] = 30.0
    state = torch.full((1, C), 7.0, device=DEV)
    got = _mingru_run(proj, (0, C, 2 * C), C, torch.zeros(C), torch.zeros(C), pieces, state, 0)
    want = _mingru_plain(proj, (0, C, 2 * C), C, torch.zeros(C), torch.zeros(C))
    u3 = float(proj[3, C])
    assert abs(float(want[399, 0]) / 30.0 - (u3 + 0.5 if u3 >= 0 else 1 / (1 + 2.718281828 ** -u3))) < 1e-6
    _close(got, want, 1e-6)
    assert float(got[:3, 0].abs().max()) < 1e-12 and float(got[:, 2].abs().max()) < 1e-12


def test_mingru_batch_of_unequal_requests_and_a_reused_slot():
    from byox_vllm_amd import kernels
    C = 48
    g = torch.Generator().manual_seed(2)
    zb, ub = torch.randn(C, generator=g), torch.randn(C, generator=g)
    seqs = {n: torch.randn(T, 3 * C, generator=g) * 2 for n, T in (("a", 37), ("b", 1), ("c", 90), ("d", 12))}
    want = {n: _mingru_plain(p, (0, C, 2 * C), C, zb, ub) for n, p in seqs.items()}
    state = torch.full((3, C), float("nan"), device=DEV)

    def launch(parts):            # parts: (name, start, count, slot)
        rows = torch.cat([seqs[n][a:a + c] for n, a, c, _ in parts]).to(DEV)
        cu = [0]
        for _, _, c, _ in parts:
            cu.append(cu[-1] + c)
        out = torch.empty(rows.size(0), C, device=DEV)
        kernels.mingru_scan(rows, (0, C, 2 * C), zb.to(DEV), ub.to(DEV), state, _i32(cu), _i32([a for _, a, _, _ in parts]),
                            _i32([s for _, _, _, s in parts]), C, out)
        for i, (n, a, c, _) in enumerate(parts):
            _close(out[cu[i]:cu[i + 1]], want[n][a:a + c], 2e-6)
    launch([("a", 0, 20, 0), ("b", 0, 1, 1), ("c", 0, 50, 2)])
    launch([("c", 50, 1, 2), ("a", 20, 17, 0), ("d", 0, 5, 1)])      # d takes the slot b has left
    launch([("d", 5, 7, 1), ("c", 51, 39, 2)])


# ------------------------------------------------------------------------------------------------ attention inside chunks
def _chunk_mask(T, chunk):
    return O.chunked(T, chunk) if chunk else O.causal(T)


def _attention_inputs(T, H, G, d, dv, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    proj = _round(torch.randn(T, (H + G) * d + G * dv + 3, generator=g), dtype)
    gate = torch.randn(T, H + 2, generator=g)
    return proj, gate, (3, 3 + H * d, 3 + (H + G) * d)


def _paged_chunk_attention(proj, offs, pieces, H, G, d, dv, scale, chunk, dtype, block, gate=None, seed=0, **store):
    """qk_rotate_store + paged_softmax_attn over one request cut into ``pieces``, on scattered pages."""
    from byox_vllm_amd import kernels
    T = proj.shape[0]
    nblocks = -(-T // block)
    g = torch.Generator().manual_seed(seed)
    pages = torch.randperm(nblocks + 3, generator=g)[:nblocks].tolist()
    cache = torch.full(((nblocks + 3) * block, G * (d + dv)), float("nan"), dtype=dtype, device=DEV)
    table = _i32([pages])
    out = torch.zeros(T, H * dv + 2, dtype=dtype, device=DEV)
    pd = proj.to(DEV)
    gd = gate.to(DEV) if gate is not None else None
    v_first = store.pop("v_first", None)
    for a, n, cu, past, _, seq_of in _steps(pieces):
        slots = _i32([pages[p // block] * block + p % block for p in range(a, a + n)])
        pos = torch.arange(a, a + n, device=DEV)
        q = kernels.qk_rotate_store(pd[a:a + n], offs, pos, scale, slots, cache, H, G, d, dv,
                                    v_first=v_first[a:a + n] if v_first is not None else None, **store)
        kernels.paged_softmax_attn(q, cache, table, cu, past, seq_of, n, H, G, d, dv, block, out[a:a + n, 2:], chunk=chunk,
                                   gate=gd[a:a + n, 2:] if gd is not None else None, gate_per_head=True)
    assert float(out[:, :2].float().abs().max()) == 0.0
    return out[:, 2:].float(), cache, pages


GEOMETRIES = [(6, 2, 16, 24, 16), (1, 1, 20, 12, 16), (3, 1, 12, 20, 32), (8, 2, 32, 32, 16), (8, 1, 128, 40, 64),
              (4, 4, 64, 16, 16), (2, 2, 24, 24, 16)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,block", GEOMETRIES)
@pytest.mark.parametrize("chunk", [20, 16, 1, 0, 1000, 7])
def test_chunked_attention_prompt_pieces_and_single_tokens(dtype, H, G, d, dv, block, chunk):
    if chunk in (1, 1000, 7) and (H, G) not in ((6, 2), (8, 2)):
        pytest.skip("the extreme chunks on two geometries")
    T = 70
    proj, gate, offs = _attention_inputs(T, H, G, d, dv, dtype, seed=H * 10 + d)
    scale = d ** -0.5
    p = proj.double()
    q, k = p[:, offs[0]:offs[0] + H * d].view(T, H, d), p[:, offs[1]:offs[1] + G * d].view(T, G, d)
    v = p[:, offs[2]:offs[2] + G * dv].view(T, G, dv)
    want = O.softmax_attention(q, k, v, scale, _chunk_mask(T, chunk)) * torch.sigmoid(gate[:, 2:].double())[:, :, None]
    want = want.reshape(T, H * dv)
    for pieces in ([T], [1] * T, [2, 2, 3, 9, 16, 1, 17, 2, 15, 3], [T - 1, 1], [33, 37]):
        got, _, _ = _paged_chunk_attention(proj, offs, pieces, H, G, d, dv, scale, chunk, dtype, block, gate)
        _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,block", [(48, 16), (64, 64), (50, 64), (16, 16)])
@pytest.mark.parametrize("pieces", [[200], [100, 100], [199, 1], [150] + [1] * 50, [97, 2, 101]])
def test_the_keys_on_both_sides_of_a_chunk_edge_stand_out(dtype, chunk, block, pieces):
    """Every position asks loudly for marked keys: head 0 for the first key of a chunk (only its own chunk's is inside),
    head 1 for the last key of a chunk (the one just outside must not be seen, whatever its score; its own chunk's last
    key is seen by the chunk's last position alone).  Head 2 has ordinary scores."""
    H, G, d, dv, T = 3, 1, 16, 8, 200
    g = torch.Generator().manual_seed(chunk)
    proj = torch.randn(T, H * d + G * d + G * dv, generator=g) * 0.2
    k_off, v_off = H * d, H * d + G * d
    for j in range(T):
        if j % chunk == 0:                    # first key of a chunk: loud on feature 0, says 1 + chunk index
            proj[j, k_off:k_off + d] = 0.0
            proj[j, k_off] = 6.0
            proj[j, v_off] = 1.0 + j // chunk
        if j % chunk == chunk - 1:            # last key of a chunk: loud on feature 1, says -50
            proj[j, k_off:k_off + d] = 0.0
            proj[j, k_off + 1] = 6.0
            proj[j, v_off + 1] = -50.0
    proj[:, 0:d], proj[:, d:2 * d] = 0.0, 0.0
    proj[:, 0], proj[:, d + 1] = 6.0, 6.0
    proj = _round(proj, dtype)
    p = proj.double()
    q, k, v = p[:, :k_off].view(T, H, d), p[:, k_off:v_off].view(T, G, d), p[:, v_off:].view(T, G, dv)
    want = O.softmax_attention(q, k, v, 1.0, O.chunked(T, chunk)).reshape(T, H * dv)
    probe = 2 * chunk + chunk // 2             # a position in the middle of the third chunk
    assert abs(float(want[probe, 0]) - 3.0) < 0.05                 # it hears its own chunk's first key ...
    assert float(want[probe, dv + 1]) > -1.0                       # ... and nothing of the key just outside
    assert float(want[3 * chunk - 1, dv + 1]) < -40.0              # its chunk's last position does hear the chunk's last key
    got, _, _ = _paged_chunk_attention(proj, (0, k_off, v_off), pieces, H, G, d, dv, 1.0, chunk, dtype, block)
    _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,rot", [(6, 2, 16, 24, 8), (1, 1, 20, 12, 20), (8, 2, 32, 32, 16), (3, 3, 12, 4, 0),
                                          (4, 1, 64, 8, 64)])
def test_norm_over_all_heads_rotation_and_value_blend(dtype, H, G, d, dv, rot):
    """What qk_rotate_store leaves as queries and in the cache rows, against the plain functions: one norm over all
    heads with a weight per number, rotation of the first ``rot`` numbers of each head at positions up to 5000, values
    blended with another layer's."""
    from byox_vllm_amd import kernels
    T, eps = 12, 1e-5
    g = torch.Generator().manual_seed(H + d)
    proj = torch.randn(T, (H + G) * d + G * dv + 3, generator=g) * 3
    offs = (3, 3 + H * d, 3 + (H + G) * d)
    qn, kn = _round(1 + 0.5 * torch.randn(H * d, generator=g), dtype), _round(1 + 0.5 * torch.randn(G * d, generator=g), dtype)
    lam = _round(torch.tensor([0.37]), dtype)
    v_first = torch.randn(T, G * dv + 1, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 17, 63, 64, 65, 1000, 4095, 4096, 5000])
    freq, mag = O.frequencies({"base": 700.0, "dims": rot}) if rot else (None, 1.0)
    cache = torch.full((T + 2, G * (d + dv)), float("nan"), dtype=dtype, device=DEV)
    slots = _i32(list(range(T - 1, -1, -1)))
    q = kernels.qk_rotate_store(proj.to(DEV), offs, pos.to(DEV), 0.3, slots, cache, H, G, d, dv, q_norm=qn.to(DEV).to(dtype),
                                k_norm=kn.to(DEV).to(dtype), eps=eps, inv_freq=freq.float().to(DEV) if rot else None,
                                rot_dims=rot, mscale=mag, v_first=v_first.to(DEV)[:, 1:], vmix=lam.to(DEV).to(dtype))
    p = proj.double()
    wq = (O.rms(p[:, offs[0]:offs[0] + H * d], eps) * qn.double()).view(T, H, d)
    wk = (O.rms(p[:, offs[1]:offs[1] + G * d], eps) * kn.double()).view(T, G, d)
    if rot:
        f32 = freq.float().double()          # the engine's table is fp32
        wq, wk = O.rotate(wq, pos, f32, mag, rot, False), O.rotate(wk, pos, f32, mag, rot, False)
    wv = (1 - lam.double()) * p[:, offs[2]:offs[2] + G * dv] + lam.double() * v_first[:, 1:].double()
    tol = (5e-4 if rot else 2e-5) if dtype == torch.float32 else 8e-3
    _close(q.view(T, H, d), wq * 0.3, 5e-4 if rot else 2e-5)      # queries stay fp32; at position 5000 a float angle is 3e-4 off
    rows = cache[:T].float().flip(0)
    _close(rows[:, :G * d].view(T, G, d), wk, tol)
    _close(rows[:, G * d:], wv, tol)
    assert torch.isnan(cache[T:].float()).all()


# ------------------------------------------------------------------------------------------------ latent attention
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,r,R", [(3, 16, 8, 32), (1, 12, 4, 20), (4, 32, 16, 64)])
def test_latent_rotation_pairs_neighbouring_dimensions(dtype, H, d, r, R):
    from byox_vllm_amd import kernels
    T, eps = 10, 1e-5
    g = torch.Generator().manual_seed(r)
    pos = torch.tensor([0, 1, 2, 5, 63, 64, 700, 1023, 1024, 4000])
    freq, mag = O.frequencies({"base": 1000.0, "dims": r, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}})
    kv = torch.randn(T, R + r, generator=g) * 2
    w = _round(1 + 0.3 * torch.randn(R, generator=g), dtype)
    cache = torch.zeros(T, R + r, dtype=dtype, device=DEV)
    kernels.latent_kv_store(kv.to(DEV), w.to(DEV).to(dtype), pos.to(DEV), freq.float().to(DEV), mag, _i32(list(range(T))),
                            cache, R, r, r, eps, interleaved=True)
    f32 = freq.float().double()
    want_k = O.rotate(kv[:, R:].double().view(T, 1, r), pos, f32, mag, r, True).view(T, r)
    tol = 2e-5 if dtype == torch.float32 else 8e-3
    _close(cache[:, :R].float(), O.rms(kv[:, :R].double(), eps) * w.double(), tol)
    _close(cache[:, R:].float(), want_k, max(tol, 5e-4))
    q = _round(torch.randn(T, H * (d + r), generator=g), dtype)
    qa = torch.zeros(T, H, R + r, device=DEV)
    kernels.latent_q_rope(q.to(DEV).to(dtype), pos.to(DEV), freq.float().to(DEV), mag, qa, H, d, r, r, R, interleaved=True)
    want_q = O.rotate(q.double().view(T, H, d + r)[..., d:], pos, f32, mag, r, True)
    _close(qa[..., R:], want_q, 5e-4)              # at position 4000 a float angle is 2e-4 off
    # the pairing differs from the half-split layout: the same call without the flag gives something else
    qb = torch.zeros(T, H, R + r, device=DEV)
    kernels.latent_q_rope(q.to(DEV).to(dtype), pos.to(DEV), freq.float().to(DEV), mag, qb, H, d, r, r, R)
    assert r < 4 or float((qa - qb).abs().max()) > 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [5, 40, 200])
@pytest.mark.parametrize("H,R,dv", [(3, 32, 24), (1, 20, 20), (4, 64, 32), (2, 256, 16)])
def test_per_number_gate_in_the_value_up_projection(dtype, rows, H, R, dv):
    """The batched per-head product with a sigmoid gate per output number, through every row-count route of nv_linear."""
    from byox_vllm_amd import kernels
    g = torch.Generator().manual_seed(rows + H)
    mix = _round(torch.randn(rows, H * R, generator=g), dtype)
    uv = _round(torch.randn(H * dv, R, generator=g) * R ** -0.5, dtype)
    logits = torch.randn(rows, 7 + H * dv, generator=g) * 2
    ld = logits.to(DEV)
    got = kernels.linear(mix.to(DEV).to(dtype), uv.to(DEV).to(dtype), batch=H, a_batch_stride=R, w_batch_stride=dv * R,
                         out_batch_stride=dv, n=dv, epilogue=kernels.EPI_ROW_GATE, act=kernels.GATE_PER_NUMBER,
                         gate=ld[:, 7:], gate_stride=ld.stride(0), out_dtype=torch.float32)
    want = torch.einsum("thr,hvr->thv", mix.double().view(rows, H, R), uv.double().view(H, dv, R)).reshape(rows, H * dv)
    _close(got, want * torch.sigmoid(logits[:, 7:].double()), 2e-5)


@pytest.mark.parametrize("rows", [100, 4200])
def test_up_projection_with_bias_and_gelu(rows):
    """Few rows take nv_linear's epilogue, thousands the vendor library and one pass over its fp32 result."""
    from byox_vllm_amd import kernels
    g = torch.Generator().manual_seed(rows)
    x = _round(torch.randn(rows, 256, generator=g), torch.bfloat16)
    w = _round(torch.randn(384, 256, generator=g) / 16, torch.bfloat16)
    b = _round(torch.randn(384, generator=g), torch.bfloat16)
    want = O.gelu_tanh(x.double() @ w.double().T + b.double())
    for out_dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 8e-3)):
        got = kernels.linear(x.to(DEV).bfloat16(), w.to(DEV).bfloat16(), b.to(DEV).bfloat16(), epilogue=kernels.EPI_ACT,
                             act=kernels.ACT_GELU_TANH, out_dtype=out_dtype)
        _close(got.float(), want, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pieces", [[600], [599, 1], [560] + [1] * 40, [300, 300]])
def test_latent_attention_hears_a_far_key_among_hundreds(dtype, pieces):
    """No window: the last position asks for key 5 among 600 (rotated parts agree at any distance only if both sides
    turn by their own positions), and the answer is that key's latent, almost alone."""
    from byox_vllm_amd import kernels
    H, R, r, T, block = 2, 32, 8, 600, 64
    g = torch.Generator().manual_seed(4)
    rows = torch.randn(T, R + r, generator=g) * 0.2
    rows[:, R:] = 0.0
    rows[5, :R] = 0.0
    rows[5, 3] = 8.0
    rows = _round(rows, dtype)
    qa = torch.randn(T, H, R + r, generator=g) * 0.2
    qa[T - 1, 0, :] = 0.0
    qa[T - 1, 0, 3] = 4.0
    nblocks = -(-T // block)
    pages = torch.randperm(nblocks + 2, generator=g)[:nblocks].tolist()
    cache = torch.zeros((nblocks + 2) * block, R + r, dtype=dtype, device=DEV)
    idx = torch.tensor([pages[p // block] * block + p % block for p in range(T)])
    cache[idx.to(DEV)] = rows.to(DEV).to(dtype)
    outs = []
    for a, n, cu, past, _, seq_of in _steps(pieces):
        outs.append(kernels.latent_attn(qa[a:a + n].contiguous().to(DEV), cache, _i32([pages]), cu, past, seq_of, H, R, r,
                                        block, 0, 1.0, max_q=n))        # single tokens: their keys split over workgroups
    got = torch.cat(outs).float().view(T, H, R)
    s = torch.einsum("thc,jc->htj", qa.double(), rows.double()).masked_fill(~O.causal(T)[None], float("-inf"))
    want = torch.einsum("htj,jc->thc", torch.softmax(s, -1), rows[:, :R].double())
    assert float(want[T - 1, 0, 3]) > 7.9                          # 32 against scores of about 0.2
    _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


# ------------------------------------------------------------------------------------------------ the engine
CASES = {"mixed": mixed_config, "odd": odd_config, "aligned": aligned_config, "plain": plain_config}


@pytest.fixture(scope="module", params=[(n, dt) for n in CASES for dt in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1])[6:]}")
def setup(request):
    name, dtype = request.param
    cfg = CASES[name]()
    weights = random_checkpoint(cfg, seed=11)
    torch.manual_seed(99)
    reqs = {"a": torch.randint(0, cfg["vocab"], (83,)).tolist(), "b": torch.randint(0, cfg["vocab"], (31,)).tolist(),
            "c": torch.randint(0, cfg["vocab"], (2,)).tolist(), "d": torch.randint(0, cfg["vocab"], (50,)).tolist()}
    want = {n: O.forward(t, weights, cfg).float() for n, t in reqs.items()}
    engine = Engine(cfg, weights, dtype, blocks=12, slots=3)
    whole = engine.replay(reqs, [[(n, len(t))] for n, t in reqs.items()])
    return cfg, weights, dtype, reqs, want, engine, whole


def _check(setup, got):
    cfg, weights, dtype, reqs, want, engine, whole = setup
    for n in got:
        if dtype == torch.float32:
            assert row_error(got[n], want[n]) < F32_TOL, (n, row_error(got[n], want[n]))
            assert row_error(got[n], whole[n]) < SAME_TOL, n
        else:
            err = row_errors(got[n], want[n])
            assert float(err.max()) < BF16_TOL, (n, float(err.max()))


def test_whole_prompts_match_the_oracle(setup):
    _check(setup, setup[6])


def test_every_layer_matches_the_oracle(setup):
    """The residual after every layer, for one request in one step (fp32 only: it is the sharp comparison)."""
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
    assert len(trace) == len(plain) == len(cfg["layers"])
    for got, ref in zip(trace, plain):
        _close(got, ref, 2e-5)


def test_prompt_then_token_by_token(setup):
    reqs = setup[3]
    # the decoded stretch crosses page borders and chunk edges
    _check(setup, setup[5].replay({"a": reqs["a"]}, [[("a", 20)]] + [[("a", 1)]] * 63))
    _check(setup, setup[5].replay({"b": reqs["b"]}, [[("b", 1)]] * 31))           # from the very first token on


def test_portions_of_many_sizes(setup):
    reqs = setup[3]
    _check(setup, setup[5].replay({"a": reqs["a"]}, [[("a", n)] for n in (2, 2, 3, 9, 16, 1, 17, 2, 15, 14, 2)]))
    _check(setup, setup[5].replay({"d": reqs["d"]}, [[("d", n)] for n in (15, 1, 16, 2, 16)]))
    _check(setup, setup[5].replay({"b": reqs["b"]}, [[("b", n)] for n in (1, 2, 1, 1, 3, 23)]))   # shorter than any tap count


def test_mixed_batches_reuse_pages_and_slots(setup):
    """Three slots, twelve pages of sixteen tokens: four requests only fit because the finished ones give theirs back.
    Prompt pieces run beside single tokens; requests sit out steps."""
    reqs = setup[3]
    schedule = [[("a", 30), ("b", 5)], [("a", 1), ("b", 20), ("c", 2)], [("a", 2), ("b", 1)], [("b", 1), ("d", 7), ("a", 1)],
                [("a", 40), ("d", 1), ("b", 4)], [("d", 30)], [("a", 1), ("d", 1)], [("a", 8), ("d", 11)]]
    _check(setup, setup[5].replay(reqs, schedule))
    # the same requests again, in slots and pages that the first pass has used
    _check(setup, setup[5].replay(reqs, [[("d", 50), ("c", 1)], [("c", 1), ("b", 31)], [("a", 83)]]))


def test_long_decoding(setup):
    """A short prompt and 170 single tokens: a dozen pages, every chunk edge of the configuration several times over."""
    cfg, weights, dtype, reqs, want, engine, whole = setup
    torch.manual_seed(7)
    tokens = torch.randint(0, cfg["vocab"], (180,)).tolist()
    got = engine.replay({"long": tokens}, [[("long", 10)]] + [[("long", 1)]] * 170)["long"]
    ref = O.forward(tokens, weights, cfg).float()
    assert row_error(got, ref) < (F32_TOL if dtype == torch.float32 else BF16_TOL), row_error(got, ref)


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
@pytest.mark.parametrize("seed", [1, 3, 4, 5, 7])
def test_drawn_configurations(seed, dtype):
    """Layer orders, sizes and constants drawn from a seed; pages of 64 tokens; prompts whole, then cut and mixed."""
    cfg = random_config(seed)
    weights = random_checkpoint(cfg, seed)
    torch.manual_seed(seed)
    reqs = {n: torch.randint(0, cfg["vocab"], (L,)).tolist() for n, L in (("a", 230), ("b", 17), ("c", 140), ("d", 2))}
    want = {n: O.forward(t, weights, cfg).float() for n, t in reqs.items()}
    engine = Engine(cfg, weights, dtype, blocks=8, slots=3, block_size=64)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    for schedule in ([[(n, len(t))] for n, t in reqs.items()],
                     [[("a", 100), ("b", 3)], [("a", 1), ("b", 14), ("d", 2)], [("a", 65), ("c", 2)], [("c", 1), ("a", 1)],
                      [("a", 63), ("c", 130)], [("c", 7)]]):
        got = engine.replay(reqs, schedule)
        for n in reqs:
            assert row_error(got[n], want[n]) < tol, (n, row_error(got[n], want[n]))
    engine.runner.exit()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_equal_eager_ones(dtype):
    """Decode steps replayed from hipGraphs (padded batches, the spare state slot, one staging copy) give the tokens of
    the eager engine, step after step, with prompt portions running eagerly between the replays."""
    from byox_vllm_amd import LLM, SamplingParams
    cfg = mixed_config()
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
