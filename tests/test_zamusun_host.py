"""Host side of the Zamusun integration on the CPU: registry and configuration, the order of layer runs, checkpoint
names and merged layouts, the cache and state specifications the engine sizes its pools from, and the oracle's own
consistency (closed forms that do not go through its loops)."""

import json
import math

import pytest
import torch

from oracle import zamusun as O
from zamusun_cases import aligned_config, looped_config, odd_config, plain_config, random_checkpoint, wide_config

F64 = torch.float64


def test_registry_and_configuration():
    from byox_vllm_amd.models import registry
    assert registry.model_class({"architecture": "Zamusun"}).__name__ == "ZamusunForCausalLM"
    cfg = looped_config()
    hf = registry.read_config(cfg, None)
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers, hf.norm_eps) == (150, 96, 4, 1e-5)
    assert (hf.loop.start, hf.loop.stop, hf.loop.times) == (1, 3, 2) and hf.tie_word_embeddings
    assert registry.read_config(plain_config(), None).loop is None
    hf.layers[0]["mixer"]["heads"] = 99                     # the given dict is left as it was
    assert cfg["layers"][0]["mixer"]["heads"] == 3
    with pytest.raises(AssertionError):
        registry.read_config(dict(cfg, loop={"start": 2, "stop": 2, "times": 2}), None)


def test_config_from_a_model_folder(tmp_path):
    from safetensors.torch import save_file

    from byox_vllm_amd.config import Config
    cfg = odd_config()
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in random_checkpoint(cfg, 1).items()}, str(tmp_path / "model.safetensors"))
    c = Config(str(tmp_path), dtype="float32", kvcache_block_size=32, max_num_seqs=3)
    assert c.portioned and c.num_state_slots == 3 and c.hf_config.dtype == torch.float32
    assert c.hf_config.layers[2]["mixer"]["gate_cap"] == 15.0


def test_order_of_layer_runs():
    from types import SimpleNamespace as NS

    from byox_vllm_amd.models.zamusun import layer_runs
    assert layer_runs(3, None) == [(0, 0, False), (1, 0, False), (2, 0, False)]
    assert layer_runs(4, NS(start=1, stop=3, times=2)) == [(0, 0, False), (1, 0, True), (2, 0, False), (1, 1, True),
                                                         (2, 1, False), (3, 0, False)]
    assert layer_runs(2, NS(start=0, stop=1, times=1)) == [(0, 0, True), (1, 0, False)]
    assert layer_runs(2, NS(start=0, stop=2, times=3)) == [(0, 0, True), (1, 0, False), (0, 1, True), (1, 1, False),
                                                         (0, 2, True), (1, 2, False)]
    for make in (looped_config, odd_config, plain_config, aligned_config):
        cfg = make()
        loop = NS(**cfg["loop"]) if "loop" in cfg else None
        assert [(i, e) for i, _, e in layer_runs(len(cfg["layers"]), loop)] == O.layer_runs(cfg)


def test_every_run_of_a_looped_layer_has_its_own_cache_and_state():
    from byox_vllm_amd.models.zamusun import ZamusunForCausalLM, zamusun_config
    m = ZamusunForCausalLM(zamusun_config(looped_config(), dtype=torch.float32))
    assert [r.page_spec()["width"] for r in m.page_layers()] == [2 * 16, 2 * 16]          # keys only: G * dim
    # mlstm: matrix + normaliser + maximum per head; lightning: the matrix alone, once per run
    assert [r.state_spec()["shape"] for r in m.state_layers()] == [(3, 16 * 24 + 16 + 1), (2, 24 * 16), (2, 24 * 16),
                                                                    (2, 8 * 40 + 8 + 1)]
    w = ZamusunForCausalLM(zamusun_config(wide_config(), dtype=torch.float32))      # 128 value columns: two slices
    assert w.state_layers()[0].state_spec()["shape"] == (1, 128 * 128 + 2 * (128 + 1))
    assert len({id(r) for r in m.page_layers() + m.state_layers()}) == 6
    p = ZamusunForCausalLM(zamusun_config(plain_config(), dtype=torch.float32))
    assert p.loop_in is None and len(p.page_layers()) == 1 and len(p.state_layers()) == 1
    a = ZamusunForCausalLM(zamusun_config(aligned_config(), dtype=torch.float32))
    assert len(a.page_layers()) == 3 and len(a.state_layers()) == 6


@pytest.mark.parametrize("make", [looped_config, odd_config, plain_config, aligned_config, wide_config])
def test_every_checkpoint_tensor_has_a_parameter_and_every_parameter_a_tensor(make):
    """Builds the model on the CPU (parameters only; nothing is launched) and loads a random checkpoint through the
    framework's loader: every tensor finds its place, merged parameters are filled completely."""
    from byox_vllm_amd.models.zamusun import ZamusunForCausalLM, zamusun_config
    from byox_vllm_amd.utils.loader import load_state_dict_packed
    cfg = make()
    weights = {k: v.float() for k, v in random_checkpoint(cfg, seed=2).items()}
    hf = zamusun_config(cfg, dtype=torch.float32)
    model = ZamusunForCausalLM(hf)
    for p in model.parameters():
        if p.dtype.is_floating_point and not (p.data == 0).all():
            p.data.fill_(float("nan"))
    load_state_dict_packed(model, weights, hf)
    for name, p in model.named_parameters():
        assert not torch.isnan(p.data).any(), name
    targets = {model.checkpoint_target(k)[0] for k in weights}
    assert targets == {n for n, _ in model.named_parameters()}
    assert model.checkpoint_target("l0.mix.nothing") is None and model.checkpoint_target("l9.norm1") is None
    # merged layouts, spot-checked
    for i, layer in enumerate(model.layers):
        mix, pre = layer.mix, f"l{i}.mix."
        if layer.kind == "attention":
            q, k, g = mix.at["q"], mix.at["k"], mix.at["g"]
            assert torch.equal(mix.inp.weight.data[k:k + mix.kv_heads * mix.dim], weights[pre + "k"])
            assert torch.equal(mix.inp.bias.data[q:q + mix.heads * mix.dim], weights[pre + "q.b"])
            assert (mix.inp.bias.data[g:] == 0).all() and torch.equal(mix.sink.data, weights[pre + "sink"])
        else:
            v = mix.at["v"]
            assert torch.equal(mix.inp.weight.data[v:v + mix.heads * mix.vdim], weights[pre + "v"])
            if layer.kind == "mlstm":
                f = mix.at["f"]
                assert torch.equal(mix.inp.bias.data[f:f + mix.heads], weights[pre + "f.b"])
                assert (mix.inp.bias.data[:mix.at["i"]] == 0).all()
        if layer.mlp is not None:
            e, ff = layer.mlp.experts - 1, layer.mlp.ff
            at, rows = mix.inp.row_of["router"]                   # the router's rows ride in the mixer's projection
            assert rows == layer.mlp.experts and at + rows == mix.inp.weight.shape[0] and layer.mlp.router is None
            assert torch.equal(mix.inp.weight.data[at:], weights[f"l{i}.mlp.router"])
            assert torch.equal(layer.mlp.gate_up.data[e, ff:], weights[f"l{i}.mlp.e{e}.up"])
            assert torch.equal(layer.mlp.down.data[0], weights[f"l{i}.mlp.e0.down"])


# ------------------------------------------------------------------------------------------------ the oracle itself
def test_lightning_equals_its_quadratic_form():
    torch.manual_seed(0)
    T, H, d, dv = 9, 2, 3, 4
    q, k, v = torch.randn(T, H, d, dtype=F64), torch.randn(T, H, d, dtype=F64), torch.randn(T, H, dv, dtype=F64)
    decay = torch.tensor([0.5, 0.9], dtype=F64)
    t = torch.arange(T)
    w = torch.where(t[:, None] >= t[None, :], decay[:, None, None] ** (t[:, None] - t[None, :]).clamp(min=0), 0.0)
    want = torch.einsum("hij,ihd,jhd,jhv->ihv", w, q, k, v)
    assert torch.allclose(O.lightning(q, k, v, decay), want, atol=1e-12)


def test_mlstm_equals_its_unstabilised_form_while_that_form_is_in_range():
    """Without the running maximum: C_t = exp(f) C + exp(i) k v^T, n likewise, o = C^T q / (max(|n . q|, 1) + 1e-6 e^m):
    the stabilised state is exp(-m) times that one, with m_0 = 0."""
    torch.manual_seed(1)
    T, H, d, dv = 12, 2, 3, 5
    q, k, v = torch.randn(T, H, d, dtype=F64), torch.randn(T, H, d, dtype=F64), torch.randn(T, H, dv, dtype=F64)
    i_log, f_log = torch.randn(T, H, dtype=F64), -torch.rand(T, H, dtype=F64)
    C, n, m = torch.zeros(H, d, dv, dtype=F64), torch.zeros(H, d, dtype=F64), torch.zeros(H, dtype=F64)
    want = []
    for t in range(T):
        C = f_log[t].exp()[:, None, None] * C + i_log[t].exp()[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = f_log[t].exp()[:, None] * n + i_log[t].exp()[:, None] * k[t]
        m = torch.maximum(f_log[t] + m, i_log[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.ones(H, dtype=F64)) + 1e-6 * m.exp()
        want.append(torch.einsum("hdv,hd->hv", C, q[t]) / den[:, None])
    assert torch.allclose(O.mlstm(q, k, v, i_log, f_log), torch.stack(want), atol=1e-10)


def test_the_sink_is_a_key_with_a_zero_value_and_an_unscaled_score():
    torch.manual_seed(2)
    T, H, G, d = 7, 4, 2, 6
    q, k = torch.randn(T, H, d, dtype=F64), torch.randn(T, G, d, dtype=F64)
    sink = torch.randn(H, dtype=F64)
    got = O.sink_attention(q, k, 0.3, sink)
    for h in range(H):
        for i in range(T):
            s = torch.cat([(k[: i + 1, h // 2] @ q[i, h]) * 0.3, sink[h: h + 1]])
            w = torch.softmax(s, 0)
            assert torch.allclose(got[i, h], (w[:-1, None] * k[: i + 1, h // 2]).sum(0), atol=1e-12)
    none = O.sink_attention(q, k, 0.3, torch.full((H,), -1e9, dtype=F64))
    assert torch.allclose(none[0], k[0].repeat_interleave(2, 0), atol=1e-12)          # one key, no sink: the key itself


def test_query_temperature_steps():
    t = O.query_temperature(40, 0.5, 16)
    assert t[14] == 1.0 and t[15] == 1.0 + 0.5 * math.log(2.0) and t[30] == t[15] and t[31] == 1.0 + 0.5 * math.log(3.0)


def test_routing_weights_and_the_clamped_unit():
    z = torch.tensor([[0.0, 2.0, 1.0, -1.0]], dtype=F64)
    idx, w = O.route(z, 2)
    assert idx.tolist() == [[1, 2]] and torch.allclose(w, torch.softmax(z[:, [1, 2]], -1))
    _, w_all = O.route(z, 4)
    assert torch.allclose(w_all.sum(), torch.tensor(1.0, dtype=F64))
    h = torch.eye(2, dtype=F64)
    gate, up, down = torch.tensor([[5.0, -1.0]], dtype=F64), torch.tensor([[-7.0, 0.5]], dtype=F64), torch.ones(1, 1, dtype=F64)
    y = O.expert(h, gate, up, down, 2.0)
    assert torch.allclose(y[0], 2.0 * torch.sigmoid(torch.tensor(3.404, dtype=F64)) * (-2.0 + 1.0))      # both clamped
    assert torch.allclose(y[1], -1.0 * torch.sigmoid(torch.tensor(-1.702, dtype=F64)) * 1.5)


def test_the_oracle_is_causal_and_the_loop_reenters_through_the_first_residual():
    cfg = looped_config()
    W = random_checkpoint(cfg, 3)
    tokens = torch.randint(0, cfg["vocab"], (20,), generator=torch.Generator().manual_seed(4)).tolist()
    full = O.forward(tokens, W, cfg)
    assert torch.allclose(O.forward(tokens[:11], W, cfg), full[:11], atol=1e-9)
    other = dict(W)
    other["loop.in"] = W["loop.in"].clone()
    other["loop.in"][:, cfg["width"]:] = 0                       # without the embedding's half the result changes
    assert not torch.allclose(O.forward(tokens, other, cfg), full, atol=1e-3)
    trace = []
    O.forward(tokens, W, cfg, trace)
    assert len(trace) == 1 + 2 * 2 + 1
