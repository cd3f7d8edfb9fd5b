"""Zamusun: a decoder-only language model of parallel blocks, x <- x + (mixer(h) + ff(h)) with h = norm1(x): one norm
feeds both sublayers.  The mixer of a layer is one of

* ``lightning``: lightning attention, a matrix memory with a constant decay per head (layers/matrix_memory.py);
* ``mlstm``: the matrix memory of xLSTM with exponential gates and a running maximum (layers/matrix_memory.py);
* ``attention``: causal softmax attention whose values are the keys, with a sink, a position-dependent query
  temperature and an output gate (layers/sink_attention.py).

The feed-forward is a mixture of experts (clamped gated units, softmax over all experts renormalised over the chosen
ones, layers/moe.py) or absent.  Norms are RMS norms with weights stored around zero (layers/hyper.py with one stream).
A span of layers ``loop.start .. loop.stop - 1`` runs ``loop.times`` times in a row with the same weights; before the
first layer of every repetition the residual is replaced by W_in [x; x0], x0 being the embedding's output, and the
repetitions keep separate cache rows and states.  The head is the embedding table.

config.json: {"architecture": "Zamusun", "vocab", "width", "norm": {"eps"}, "loop": {"start", "stop", "times"} | absent,
"layers": [{"type", "mixer": {...}, "mlp": {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff", "limit"}} |
null}]}.  Checkpoint tensor names: 'embed', 'loop.in', 'final.norm', 'l<i>.norm1', 'l<i>.mix.<name>[.b]',
'l<i>.mlp.router', 'l<i>.mlp.e<k>.gate|up|down'.

The residual is fp32 from the embedding to the final norm.  The model steps through portions: any mixture of prompt
pieces and single decoded tokens in one batch, each request continuing from its pages and its state slot
(engine/model_runner.py run_portions)."""

import json
import re
from types import SimpleNamespace

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.hyper import StreamNorm
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.layers.matrix_memory import MLSTM, LightningAttention
from byox_vllm_amd.layers.moe import MixtureOfExperts
from byox_vllm_amd.layers.sink_attention import SinkAttention


def zamusun_config(raw: dict, dtype=torch.bfloat16):
    """config.json contents -> the configuration object the engine and the model read."""
    layers = json.loads(json.dumps(raw["layers"]))           # deep copy
    loop = raw.get("loop")
    if loop:
        loop = SimpleNamespace(start=int(loop["start"]), stop=int(loop["stop"]), times=int(loop["times"]))
        assert 0 <= loop.start < loop.stop <= len(layers) and loop.times >= 1, f"bad loop {raw['loop']}"
    return SimpleNamespace(
        architecture="Zamusun", vocab_size=raw["vocab"], hidden_size=raw["width"],
        norm_eps=float((raw.get("norm") or {}).get("eps", 1e-6)), loop=loop or None,
        layers=layers, num_hidden_layers=len(layers), max_position_embeddings=1 << 30, dtype=dtype,
        tie_word_embeddings=True)


def layer_runs(n_layers: int, loop) -> list:
    """The order in which layers run: (layer, which of the layer's runs this is, does a pass of the loop begin here)."""
    if loop is None:
        return [(i, 0, False) for i in range(n_layers)]
    runs = [(i, 0, False) for i in range(loop.start)]
    for r in range(loop.times):
        runs += [(i, r, i == loop.start) for i in range(loop.start, loop.stop)]
    return runs + [(i, 0, False) for i in range(loop.stop, n_layers)]


class ZamusunLayer(nn.Module):
    def __init__(self, cfg, spec: dict, runs: int):
        super().__init__()
        width, eps, m = cfg.hidden_size, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        self.norm1 = StreamNorm(width, 1, eps, connections=False)
        mlp = spec.get("mlp")
        if mlp and mlp["kind"] != "moe":
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        # mixer and router read the same rows: the router's rows ride in the mixer's input projection
        riders = {"router": mlp["router"]["experts"]} if mlp else None
        if self.kind == "lightning":
            self.mix = LightningAttention(width, m["heads"], m["dim"], m["vdim"], m["decay"], eps, runs, riders)
        elif self.kind == "mlstm":
            self.mix = MLSTM(width, m["heads"], m["dim"], m["vdim"], m["gate_cap"], eps, runs, riders)
        elif self.kind == "attention":
            assert m.get("vdim", m["dim"]) == m["dim"], "the values are the keys: they have the keys' size"
            temp = m.get("q_temp") or {}
            self.mix = SinkAttention(width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["scale"],
                                     temp.get("coef", 0.0), temp.get("every", 0), runs, riders)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.mlp = None
        if mlp:
            self.mlp = MixtureOfExperts(width, mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"],
                                        "clamped", route="all", limit=mlp["expert"]["limit"], own_router=False)

    def forward(self, x, delta, positions, run: int):
        """x: fp32 residual [T, width] (updated in place by ``delta``, what the previous layer still owes it) -> what
        this layer owes it: mixer and feed-forward of the same normed rows, summed."""
        h = self.norm1(x.unsqueeze(1), (delta, None) if delta is not None else None)
        proj = self.mix.project(h)
        y = self.mix(h, run, positions, proj)
        return self.mlp(h, add=y, logits=self.mix.rider(proj, "router")) if self.mlp is not None else y


class ZamusunForCausalLM(nn.Module):
    portioned = True          # steps through ModelRunner.run_portions: prompt pieces and decoded tokens in one batch
    prefix_cache = False      # a recurrent state cannot be rebuilt from cached pages
    kernel_sources = ("linear", "rowops", "streams", "window_attn", "memory", "moe", "misc", "gemm_lt")

    @staticmethod
    def config_from_json(raw: dict, path: str | None):
        return zamusun_config(raw)

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        width, loop = cfg.hidden_size, cfg.loop
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, width), requires_grad=False)
        self.order = layer_runs(len(cfg.layers), loop)
        self.layers = nn.ModuleList(
            ZamusunLayer(cfg, spec, loop.times if loop is not None and loop.start <= i < loop.stop else 1)
            for i, spec in enumerate(cfg.layers))
        self.loop_in = DenseLinear(2 * width, width) if loop is not None else None
        self.final_norm = StreamNorm(width, 1, cfg.norm_eps, connections=False)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace: list | None = None):
        """-> (fp32 residual [T, width], what the last layer still owes it).  ``trace`` collects the residual after
        every layer run (a debugging aid: it adds the pending output eagerly)."""
        x = kernels.embed_scale(input_ids, self.embed.data, 1.0)
        x0 = x.clone() if self.loop_in is not None else None          # x is updated in place from here on
        delta = None
        for i, run, enters in self.order:
            if enters:
                pair = kernels.residual_pair(x, x0, self.embed.dtype, delta)
                x, delta = self.loop_in(pair, out_dtype=torch.float32), None
            delta = self.layers[i](x, delta, positions, run)
            if trace is not None:
                x += delta
                delta = None
                trace.append(x.clone())
        return x, delta

    def compute_logits(self, state, rows_idx=None, out_dtype=torch.float32):
        """Final norm on the wanted rows, then the embedding table as the head -> logits [rows, vocab]."""
        x, delta = state
        if rows_idx is None:
            rows_idx = torch.arange(x.size(0), dtype=torch.int32, device=x.device)
        h = self.final_norm(x.unsqueeze(1), (delta, None) if delta is not None else None, rows_idx)
        return kernels.linear(h, self.embed.data, out_dtype=out_dtype)

    def finalize(self, quantization=None) -> None:
        assert quantization is None, "Zamusun runs unquantised"

    # ------------------------------------------------------------------ cache and state
    def page_layers(self):
        """Holders of paged cache rows: one per run of every attention layer."""
        return [run for l in self.layers if l.kind == "attention" for run in l.mix.runs]

    def state_layers(self):
        """Holders of a piece of a request's state slot: one per run of every matrix-memory layer."""
        return [run for l in self.layers if l.kind != "attention" for run in l.mix.state_modules()]

    # ------------------------------------------------------------------ checkpoint names
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")
    _EXPERT = re.compile(r"^e(\d+)\.(gate|up|down)$")
    _MEMORY = {"q": ("inp.weight", "q"), "k": ("inp.weight", "k"), "v": ("inp.weight", "v"), "g": ("inp.weight", "g"),
               "norm": ("norm", None), "o": ("o.weight", None)}
    _MLSTM = dict(_MEMORY, **{"i": ("inp.weight", "i"), "f": ("inp.weight", "f"), "i.b": ("inp.bias", "i"),
                              "f.b": ("inp.bias", "f")})
    _ATTENTION = {"q": ("inp.weight", "q"), "k": ("inp.weight", "k"), "g": ("inp.weight", "g"), "q.b": ("inp.bias", "q"),
                  "k.b": ("inp.bias", "k"), "sink": ("sink", None), "o": ("o.weight", None), "o.b": ("o.bias", None)}

    def checkpoint_target(self, name: str):
        """Checkpoint tensor name -> (parameter path, shard id or None); None for a name this model does not own."""
        if name == "embed":
            return "embed", None
        if name == "final.norm":
            return "final_norm.weight", None
        if name == "loop.in":
            return ("loop_in.weight", None) if self.loop_in is not None else None
        m = self._LAYER.match(name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None
        i, rest = int(m.group(1)), m.group(2)
        base = f"layers.{i}."
        layer = self.layers[i]
        if rest == "norm1":
            return base + "norm1.weight", None
        part, _, leaf = rest.partition(".")
        if part == "mix":
            table = {"lightning": self._MEMORY, "mlstm": self._MLSTM, "attention": self._ATTENTION}[layer.kind]
            return (base + "mix." + table[leaf][0], table[leaf][1]) if leaf in table else None
        if part == "mlp" and layer.mlp is not None:
            if leaf == "router":
                return base + "mix.inp.weight", "router"
            e = self._EXPERT.match(leaf)
            if e and int(e.group(1)) < layer.mlp.experts:
                if e.group(2) == "down":
                    return base + "mlp.down", int(e.group(1))
                return base + "mlp.gate_up", (int(e.group(1)), e.group(2))
        return None
