"""Kikelorn: a decoder-only language model whose sublayers carry their norm on the OUTPUT, read the residual through a
short causal convolution, and are gated by the residual itself (layers/postnorm.py):

    y = f(x + conv(x)),   x <- x + m * rms_norm(y * sigmoid(W_r x + b_r)) * w          m = residual_mult

first with f = the layer's mixer, then with f = its feed-forward.  The mixer of a layer is one of

* ``attention``: grouped softmax attention inside chunks of the sequence, with a short convolution behind q, k and v,
  one RMS norm over all heads of q and of k, a partial rotation, values blended with those of the first layer that
  shares its values, and one gate number per head (layers/chunked_attention.py);
* ``latent_attention``: causal attention over a cache of low-rank latents with a rotated key part shared by the heads,
  pairs of neighbouring dimensions rotated together, frequencies scaled in the YaRN manner, and a gate number per output
  number (layers/latent_attention.py);
* ``mingru``: the minimal gated recurrent unit (layers/mingru.py).

Feed-forwards are W_down gelu(W_up h + b) + b (layers/mlp.py) or absent.  The embedding is scaled; the head is the
embedding table without the scale, behind a final RMS norm.

config.json: {"architecture": "Kikelorn", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"}, "residual_mult",
"canon": {"taps"}, "layers": [{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}]}.  Checkpoint tensor
names: 'embed', 'final.norm', 'l<i>.norm1|norm2', 'l<i>.canon1|canon2', 'l<i>.rg1|rg2[.b]', 'l<i>.mix.<name>',
'l<i>.mlp.up|down[.b]'.

The residual is fp32 from the embedding to the final norm.  The model steps through portions: any mixture of prompt
pieces and single decoded tokens in one batch, each request continuing from its pages and its state slot
(engine/model_runner.py run_portions)."""

import json
import re
from types import SimpleNamespace

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.chunked_attention import ChunkedAttention
from byox_vllm_amd.layers.hyper import StreamNorm
from byox_vllm_amd.layers.latent_attention import LatentAttention
from byox_vllm_amd.layers.mingru import MinGRU
from byox_vllm_amd.layers.mlp import UnaryMLP
from byox_vllm_amd.layers.postnorm import GatedPostNorm, fold


def kikelorn_config(raw: dict, dtype=torch.bfloat16):
    """config.json contents -> the configuration object the engine and the model read."""
    layers = json.loads(json.dumps(raw["layers"]))           # deep copy
    return SimpleNamespace(
        architecture="Kikelorn", vocab_size=raw["vocab"], hidden_size=raw["width"],
        embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
        norm_eps=float((raw.get("norm") or {}).get("eps", 1e-6)), residual_mult=float(raw.get("residual_mult", 1.0)),
        canon_taps=int((raw.get("canon") or {}).get("taps", 0)),
        layers=layers, num_hidden_layers=len(layers), max_position_embeddings=1 << 30, dtype=dtype,
        tie_word_embeddings=True)


class KikelornLayer(nn.Module):
    def __init__(self, cfg, spec: dict, earlier: list):
        super().__init__()
        width, eps, m = cfg.hidden_size, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        self.norm1 = GatedPostNorm(width, eps, cfg.residual_mult, cfg.canon_taps)
        rot = m.get("rot") or {}
        if self.kind == "attention":
            first = None
            if m.get("v_mix"):       # the first layer that shares its values lends them to the later ones
                first = next((l.mix for l in earlier if l.kind == "attention" and l.mix.keeps_values), None)
            self.mix = ChunkedAttention(width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"], m["scale"],
                                        int((m.get("mask") or {}).get("size", 0)), int(m.get("conv") or 0),
                                        int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), rot.get("scaling"),
                                        eps, v_source=first, keeps_values=bool(m.get("v_mix")) and first is None)
        elif self.kind == "latent_attention":
            self.mix = LatentAttention(width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"],
                                       float(m["scale"]), int((m.get("mask") or {}).get("size", 0)), m["rot_dim"],
                                       float(rot.get("base", 10000.0)), rot.get("scaling"), eps, interleaved=True,
                                       gate="channel")
        elif self.kind == "mingru":
            self.mix = MinGRU(width, m["width"])
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        self.norm2 = self.mlp = None
        if mlp:
            if mlp["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            self.norm2 = GatedPostNorm(width, eps, cfg.residual_mult, cfg.canon_taps)
            self.mlp = UnaryMLP(width, mlp["ff"], "gelu_tanh", bias=True)

    def forward(self, x, pending, positions):
        """x: fp32 residual [T, width] (updated in place); pending: what the previous sublayer still owes it
        -> what this layer's last sublayer owes it."""
        h, logits = self.norm1.begin(x, pending)
        y = self.mix(h) if self.kind == "mingru" else self.mix(h, positions)
        pending = (y, logits, self.norm1)
        if self.mlp is not None:
            h, logits = self.norm2.begin(x, pending)
            y, y_bias = self.mlp(h, defer_bias=True)
            pending = (y, logits, self.norm2, y_bias)
        return pending


class KikelornForCausalLM(nn.Module):
    portioned = True          # steps through ModelRunner.run_portions: prompt pieces and decoded tokens in one batch
    prefix_cache = False      # a recurrent state cannot be rebuilt from cached pages
    kernel_sources = ("linear", "rowops", "streams", "window_attn", "latent_attn", "scan", "misc", "gemm_lt")

    @staticmethod
    def config_from_json(raw: dict, path: str | None):
        return kikelorn_config(raw)

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size), requires_grad=False)
        self.layers = nn.ModuleList()
        for spec in cfg.layers:
            self.layers.append(KikelornLayer(cfg, spec, list(self.layers)))
        self.final_norm = StreamNorm(cfg.hidden_size, 1, cfg.norm_eps, connections=False, one_plus=False)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace: list | None = None):
        """-> (fp32 residual [T, width], what the last sublayer still owes it).  ``trace`` collects the residual after
        every layer (a debugging aid: it adds the pending result eagerly)."""
        x = kernels.embed_scale(input_ids, self.embed.data, self.cfg.embedding_scale)
        pending = None
        for layer in self.layers:
            pending = layer(x, pending, positions)
            if trace is not None:
                fold(x, pending)
                pending = None
                trace.append(x.clone())
        return x, pending

    def compute_logits(self, state, rows_idx=None, out_dtype=torch.float32):
        """Final norm on the wanted rows, then the embedding table as the head -> logits [rows, vocab]."""
        x, pending = state
        fold(x, pending)
        if rows_idx is None:
            rows_idx = torch.arange(x.size(0), dtype=torch.int32, device=x.device)
        h = self.final_norm(x.unsqueeze(1), None, rows_idx)
        return kernels.linear(h, self.embed.data, out_dtype=out_dtype)

    def finalize(self, quantization=None) -> None:
        assert quantization is None, "Kikelorn runs unquantised"

    # ------------------------------------------------------------------ cache and state
    def page_layers(self):
        """Mixers that own rows of the paged cache."""
        return [l.mix for l in self.layers if l.kind in ("attention", "latent_attention")]

    def state_layers(self):
        """Modules that own a piece of a request's state slot: every sublayer's input convolution, the attention's
        convolution over q | k | v, the recurrence."""
        out = []
        for l in self.layers:
            out.extend(l.norm1.state_modules())
            if l.kind != "latent_attention":
                out.extend(l.mix.state_modules())
            if l.norm2 is not None:
                out.extend(l.norm2.state_modules())
        return out

    # ------------------------------------------------------------------ checkpoint names
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")
    _ATTENTION = {"q": ("inp.weight", "q"), "k": ("inp.weight", "k"), "v": ("inp.weight", "v"), "g": ("inp.weight", "g"),
                  "q.conv": ("conv.weight", "q"), "k.conv": ("conv.weight", "k"), "v.conv": ("conv.weight", "v"),
                  "q.norm": ("q_norm", None), "k.norm": ("k_norm", None), "vmix": ("vmix", None), "o": ("o.weight", None)}
    _LATENT = {"dq": ("down.weight", "dq"), "dkv": ("down.weight", "dkv"), "g": ("down.weight", "g"),
               "dq.norm": ("dq_norm", None), "dkv.norm": ("dkv_norm", None), "uq": ("uq.weight", None),
               "uk": ("uk_t", None), "uv": ("uv.weight", None), "o": ("o.weight", None)}
    _MINGRU = {"z": ("inp.weight", "z"), "x": ("inp.weight", "x"), "g": ("inp.weight", "g"), "z.b": ("z_bias", None),
               "x.b": ("x_bias", None), "o": ("o.weight", None)}
    _SUBLAYER = {"norm": "weight", "canon": "conv.weight", "rg": "gate.weight", "rg.b": "gate.bias"}

    def checkpoint_target(self, name: str):
        """Checkpoint tensor name -> (parameter path, shard id or None); (None, None) for a tensor the configuration
        leaves without a consumer; None for a name this model does not own."""
        if name == "embed":
            return "embed", None
        if name == "final.norm":
            return "final_norm.weight", None
        m = self._LAYER.match(name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None
        i, rest = int(m.group(1)), m.group(2)
        base = f"layers.{i}."
        layer = self.layers[i]
        s = re.match(r"^(norm|canon|rg)([12])(\.b)?$", rest)
        if s:
            norm = getattr(layer, "norm" + s.group(2))
            key = s.group(1) + (s.group(3) or "")
            if key not in self._SUBLAYER:
                return None
            if norm is None or (s.group(1) == "canon" and norm.conv is None):
                return None, None
            return f"{base}norm{s.group(2)}.{self._SUBLAYER[key]}", None
        part, _, leaf = rest.partition(".")
        if part == "mix":
            table = {"attention": self._ATTENTION, "latent_attention": self._LATENT, "mingru": self._MINGRU}[layer.kind]
            if leaf not in table:
                return None
            target, shard = table[leaf]
            if layer.kind == "attention":
                if (leaf == "vmix" and layer.mix.vmix is None) or (leaf.endswith(".conv") and layer.mix.conv is None):
                    return None, None
            return base + "mix." + target, shard
        if part == "mlp":
            if layer.mlp is None:
                return None, None
            table = {"up": "up.weight", "up.b": "up.bias", "down": "down.weight", "down.b": "down.bias"}
            return (base + "mlp." + table[leaf], None) if leaf in table else None
        return None
