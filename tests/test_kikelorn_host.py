"""Host side of the Kikelorn integration on the CPU: registry and configuration, checkpoint names and merged layouts,
the cache and state specifications the engine sizes its pools from, rotation frequencies, and the oracle's own
consistency (closed forms that do not go through its loops)."""

import json
import math

import torch

from kikelorn_cases import aligned_config, mixed_config, odd_config, plain_config, random_checkpoint
from oracle import kikelorn as O

F64 = torch.float64


def _model(cfg, dtype=torch.bfloat16):
    from byox_vllm_amd.models.kikelorn import KikelornForCausalLM, kikelorn_config
    default = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        return KikelornForCausalLM(kikelorn_config(cfg, dtype=dtype))
    finally:
        torch.set_default_dtype(default)


def test_registry_and_configuration():
    from byox_vllm_amd.models import registry
    assert registry.model_class({"architecture": "Kikelorn"}).__name__ == "KikelornForCausalLM"
    cfg = mixed_config()
    hf = registry.read_config(cfg, None)
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers, hf.norm_eps) == (150, 96, 5, 1e-5)
    assert (hf.residual_mult, hf.embedding_scale, hf.canon_taps) == (0.7, 1.5, 4) and hf.tie_word_embeddings
    assert registry.read_config(plain_config(), None).canon_taps == 0
    hf.layers[1]["mixer"]["heads"] = 99                     # the given dict is left as it was
    assert cfg["layers"][1]["mixer"]["heads"] == 6


def test_config_from_a_model_folder(tmp_path):
    from safetensors.torch import save_file

    from byox_vllm_amd.config import Config
    cfg = odd_config()
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in random_checkpoint(cfg, 1).items()}, str(tmp_path / "model.safetensors"))
    c = Config(str(tmp_path), dtype="float32", kvcache_block_size=32, max_num_seqs=3)
    assert c.portioned and c.num_state_slots == 3 and c.hf_config.dtype == torch.float32
    assert c.hf_config.layers[2]["mixer"]["width"] == 36


def test_every_checkpoint_tensor_has_a_parameter_and_every_parameter_a_tensor():
    from byox_vllm_amd.utils.loader import load_state_dict_packed
    for make in (mixed_config, odd_config, aligned_config, plain_config):
        cfg = make()
        W = random_checkpoint(cfg, 3)
        model = _model(cfg)
        for p in model.parameters():
            p.data.fill_(float("nan"))
        load_state_dict_packed(model, W, model.cfg)
        unused = [n for n, p in model.named_parameters() if torch.isnan(p.float()).any()]
        assert not unused, unused
        assert model.checkpoint_target("l0.mix.nothing") is None and model.checkpoint_target("l99.norm1") is None
        assert model.checkpoint_target("head") is None


def test_merged_layouts():
    cfg = mixed_config()
    W = random_checkpoint(cfg, 4)
    from byox_vllm_amd.utils.loader import load_state_dict_packed
    model = _model(cfg)
    load_state_dict_packed(model, W, model.cfg)
    att = model.layers[1].mix                                # 6 query heads on 2 key heads of 16, values of 24
    assert att.inp.weight.shape == (6 * 16 + 2 * 16 + 2 * 24 + 6, 96)
    assert torch.equal(att.inp.weight[96:128], W["l1.mix.k"]) and torch.equal(att.inp.weight[-6:], W["l1.mix.g"])
    assert torch.equal(att.conv.weight[128:176], W["l1.mix.v.conv"]) and att.conv.bias is None
    assert att.keeps_values and att.v_source is None and model.layers[3].mix.v_source is att
    assert float(model.layers[3].mix.vmix) == float(W["l3.mix.vmix"])
    lat = model.layers[2].mix                                # W_uk per head, transposed
    assert torch.equal(lat.uk_t[1], W["l2.mix.uk"][16:32].T) and lat.down.weight.shape == (40 + 32 + 8 + 3 * 24, 96)
    gru = model.layers[0].mix
    assert torch.equal(gru.inp.weight[80:160], W["l0.mix.x"]) and torch.equal(gru.z_bias, W["l0.mix.z.b"])
    assert torch.equal(model.layers[0].norm2.gate.bias, W["l0.rg2.b"])
    assert torch.equal(model.layers[4].norm1.conv.weight, W["l4.canon1"]) and model.layers[4].norm2 is None
    # a layer without input convolution skips its tensor, should a checkpoint carry one
    assert _model(plain_config()).checkpoint_target("l0.canon1") == (None, None)


def test_pool_specifications():
    model = _model(mixed_config())
    assert [m.page_spec()["width"] for m in model.page_layers()] == [2 * (16 + 24), 32 + 8, 2 * (24 + 24)]
    shapes = [tuple(m.state_spec()["shape"]) for m in model.state_layers()]
    # per layer: the mixer's input convolution, the mixer's own state, the feed-forward's input convolution
    assert shapes == [(3, 96), (80,), (3, 96),
                      (3, 96), (2, 176), (3, 96),
                      (3, 96),
                      (3, 96), (1, 144), (3, 96),
                      (3, 96), (50,)]
    plain = _model(plain_config())                           # no input convolutions: only the mixers keep state
    assert [tuple(m.state_spec()["shape"]) for m in plain.state_layers()] == [(3, 8 * 128 + 128 + 40), (64,)]
    one = _model(odd_config())                               # one tap: a state of no rows
    assert tuple(one.state_layers()[0].state_spec()["shape"]) == (0, 100)


def test_rotation_frequencies_match_the_oracle():
    from byox_vllm_amd.layers.rotary_embedding import scaled_inv_freq
    for rot in ({"base": 10000.0, "dims": 16}, {"base": 500.0, "dims": 8},
                {"base": 3000.0, "dims": 8, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}},
                {"base": 1e6, "dims": 64, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
                {"base": 50.0, "dims": 4, "scaling": {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}}):
        f, mag = scaled_inv_freq(rot["dims"], rot["base"], rot.get("scaling"))
        want, wmag = O.frequencies(rot)
        assert torch.allclose(f.double(), want, rtol=1e-6, atol=0) and abs(mag - wmag) < 1e-12
    f, mag = O.frequencies({"base": 1e6, "dims": 64, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}})
    plain = 1e6 ** (-2.0 * torch.arange(32, dtype=F64) / 64)
    assert torch.equal(f[:5], plain[:5]) and torch.allclose(f[-3:], plain[-3:] / 4.0) and abs(mag - (0.1 * math.log(4) + 1)) < 1e-12
    assert bool(((f <= plain) & (f >= plain / 4.0)).all())


# ------------------------------------------------------------------------------------------------ the oracle itself
def test_oracle_is_causal_and_chunks_forget():
    cfg = mixed_config()
    W = random_checkpoint(cfg, 5)
    torch.manual_seed(0)
    a = torch.randint(0, cfg["vocab"], (30,)).tolist()
    b = list(a)
    b[25] = (b[25] + 1) % cfg["vocab"]
    la, lb = O.forward(a, W, cfg), O.forward(b, W, cfg)
    assert torch.equal(la[:25], lb[:25]) and not torch.equal(la[25:], lb[25:])


def test_chunk_mask():
    m = O.chunked(10, 4)
    assert m[5].tolist() == [False] * 4 + [True, True] + [False] * 4           # position 5: keys 4 and 5
    assert m[4].tolist() == [False] * 4 + [True] + [False] * 5                  # a chunk's first position sees itself alone
    assert m[3].tolist() == [True] * 4 + [False] * 6
    assert torch.equal(O.chunked(10, 100), O.causal(10)) and torch.equal(O.chunked(6, 1), torch.eye(6, dtype=torch.bool))


def test_rotation_keeps_lengths_and_depends_on_distance_only():
    g = torch.Generator().manual_seed(0)
    x, y = torch.randn(1, 1, 12, generator=g, dtype=F64), torch.randn(1, 1, 12, generator=g, dtype=F64)
    f, _ = O.frequencies({"base": 100.0, "dims": 8})
    for inter in (False, True):
        dots = []
        for p in (0, 7, 1000):
            a = O.rotate(x, torch.tensor([p + 5]), f, 1.0, 8, inter)
            b = O.rotate(y, torch.tensor([p]), f, 1.0, 8, inter)
            assert abs(float(a.norm()) - float(x.norm())) < 1e-12 and torch.equal(a[..., 8:], x[..., 8:])
            dots.append(float((a * b).sum()))
        assert max(dots) - min(dots) < 1e-9
    half, inter = O.rotate(x, torch.tensor([3]), f, 1.0, 8, False), O.rotate(x, torch.tensor([3]), f, 1.0, 8, True)
    assert not torch.allclose(half, inter)
    # the interleaved layout is the half-split one on permuted dimensions
    perm = [0, 2, 4, 6, 1, 3, 5, 7]
    xp = x.clone()
    xp[..., :8] = x[..., perm]
    back = O.rotate(xp, torch.tensor([3]), f, 1.0, 8, False)
    assert torch.allclose(back[..., :8], inter[..., perm])


def test_min_gru_closed_form():
    """With a constant gate z and a constant candidate c the state is c (1 - (1 - z)^t)."""
    z, u = torch.full((20, 1), 0.3, dtype=F64), torch.full((20, 1), 1.5, dtype=F64)
    S = O.min_gru(z, u)[:, 0]
    t = torch.arange(1, 21, dtype=F64)
    assert torch.allclose(S, 2.0 * (1 - 0.7 ** t))
    S = O.min_gru(z, -u)[:, 0]
    assert torch.allclose(S, torch.sigmoid(torch.tensor(-1.5, dtype=F64)) * (1 - 0.7 ** t))


def test_latent_attention_equals_attention_over_expanded_keys():
    """Folding W_uk into the query and applying W_uv after the weighted sum of latents changes nothing."""
    cfg = aligned_config()
    W = {k: v.to(F64) for k, v in random_checkpoint(cfg, 6).items()}
    m = cfg["layers"][1]["mixer"]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = 9
    h = torch.randn(T, cfg["width"], dtype=F64, generator=torch.Generator().manual_seed(1))
    want = O.latent_attention_mixer(h, W, "l1.mix.", m, 1e-5, {})
    cq = O.rms(h @ W["l1.mix.dq"].T, 1e-5) * W["l1.mix.dq.norm"]
    q = (cq @ W["l1.mix.uq"].T).view(T, H, d + r)
    down = h @ W["l1.mix.dkv"].T
    c = O.rms(down[:, :R], 1e-5) * W["l1.mix.dkv.norm"]
    f, mag = O.frequencies(dict(m["rot"], dims=r))
    pos = torch.arange(T)
    q_rot, k_rot = O.rotate(q[..., d:], pos, f, mag, r, True), O.rotate(down[:, R:].view(T, 1, r), pos, f, mag, r, True)
    qa = torch.einsum("thd,hdc->thc", q[..., :d], W["l1.mix.uk"].view(H, d, R))
    s = (torch.einsum("thc,jc->htj", qa, c) + torch.einsum("thr,jr->htj", q_rot, k_rot[:, 0])) * m["scale"]
    p = torch.softmax(s.masked_fill(~O.causal(T)[None], float("-inf")), -1)
    o = torch.einsum("thc,hvc->thv", torch.einsum("htj,jc->thc", p, c), W["l1.mix.uv"].view(H, dv, R)).reshape(T, H * dv)
    got = (o * torch.sigmoid(h @ W["l1.mix.g"].T)) @ W["l1.mix.o"].T
    assert torch.allclose(got, want, rtol=1e-9, atol=1e-9)


def test_the_first_sharing_layer_lends_its_values():
    """Changing the second sharing layer's blend weight to zero must cut the path from the first layer's values."""
    cfg = mixed_config()
    W = random_checkpoint(cfg, 7)
    toks = list(range(12))
    base = O.forward(toks, W, cfg)
    W2 = dict(W)
    W2["l1.mix.vmix"] = torch.tensor(0.9, dtype=torch.bfloat16)      # the first layer's own number is never read
    assert torch.equal(O.forward(toks, W2, cfg), base)
    W3 = dict(W)
    W3["l3.mix.vmix"] = torch.tensor(0.0, dtype=torch.bfloat16)
    assert not torch.equal(O.forward(toks, W3, cfg), base)
