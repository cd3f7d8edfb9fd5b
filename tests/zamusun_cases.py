"""Small Zamusun configurations, helpers and an engine harness shared by the host and GPU tests.  Sizes are deliberately
awkward: key and value sizes that differ, head counts that are no powers of two, widths that are no multiples of 8,
several query heads per key head and one, a looped span that starts after the first layer and one that covers every
layer, a span that runs once, no loop at all, one expert per token and every expert per token, a layer without a
feed-forward, a query temperature whose steps fall inside the prompts."""

import copy

import torch

from oracle import zamusun as O


def mlstm(heads, dim, vdim, cap=10.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def lightning(heads, dim, vdim, decay):
    assert len(decay) == heads
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def attention(heads, kv_heads, dim, scale, coef=None, every=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if coef is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def config(vocab, width, layers, loop=None, eps=1e-5):
    cfg = {"architecture": "Zamusun", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [dict(copy.deepcopy(mixer), mlp=mlp) for mixer, mlp in layers]}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def looped_config():
    """The span starts after the first layer and holds an attention layer (two caches) and a lightning layer (two
    states); three query heads per key head; the temperature steps every 16 positions; one layer has no feed-forward."""
    return config(150, 96, [
        (mlstm(3, 16, 24), moe(5, 2, 40, 1.5)),
        (attention(6, 2, 16, 0.2, 0.4, 16), moe(4, 3, 24, 2.5)),
        (lightning(2, 24, 16, [0.7, 0.96]), None),
        (mlstm(2, 8, 40, 6.0), moe(6, 2, 32, 1.0)),
    ], loop=(1, 3, 2))


def odd_config():
    """Nothing is a multiple of 8; single heads; one expert per token; the span is the first layer alone and runs once
    (the re-entry projection is still applied); no temperature."""
    return config(77, 100, [
        (lightning(1, 12, 20, [0.9]), moe(3, 1, 36, 3.0)),
        (attention(1, 1, 20, 0.3), moe(2, 2, 28, 0.7)),
        (mlstm(1, 20, 12, 15.0), None),
    ], loop=(0, 1, 1), eps=1e-6)


def plain_config():
    """No loop entry and no 'loop.in' tensor; every expert is chosen (the weights are the softmax itself)."""
    return config(64, 48, [
        (attention(4, 4, 8, 0.35, 1.5, 5), moe(3, 3, 16, 2.0)),
        (lightning(3, 8, 8, [0.5, 0.9, 0.999]), moe(4, 1, 24, 2.0)),
    ])


def aligned_config():
    """Sizes in multiples of 16 and 32, where the 16-bit engine takes its matrix-core kernels; the span covers every
    layer and runs three times."""
    return config(256, 128, [
        (mlstm(2, 64, 64), moe(8, 2, 48, 2.5)),
        (attention(8, 2, 32, 32 ** -0.5, 0.25, 32), moe(4, 2, 96, 4.0)),
        (lightning(2, 64, 32, [0.75, 0.995]), None),
    ], loop=(0, 3, 3))


def wide_config():
    """States of 128 x 128 and 128 x 32 numbers per head; eight query heads on one key head of 128."""
    return config(90, 64, [
        (mlstm(1, 128, 128, 8.0), None),
        (attention(8, 1, 128, 0.09), moe(2, 1, 48, 2.0)),
        (lightning(2, 128, 32, [0.8, 0.99]), None),
    ], loop=(1, 2, 2))


def random_checkpoint(cfg, seed=0):
    return O.random_weights(cfg, seed)


def engine_config(cfg_json, weights, dtype, blocks=16, slots=4, block_size=16, **kw):
    """The engine's Config for an in-memory checkpoint of one of the configurations above."""
    from byox_vllm_amd.config import Config
    from byox_vllm_amd.models.zamusun import zamusun_config
    hf = zamusun_config(cfg_json, dtype=dtype)
    return Config("synthetic", hf_config=hf, state_dict=weights, kvcache_block_size=block_size, num_kvcache_blocks=blocks,
                  max_num_seqs=slots, num_state_slots=slots, enforce_eager=True, max_num_batched_tokens=1 << 20,
                  max_model_len=1 << 20, **kw)


class Engine:
    """ModelRunner + Scheduler of one configuration, replaying schedules of (request name, token count) steps."""

    def __init__(self, cfg_json, weights, dtype, blocks=16, slots=4, block_size=16):
        from byox_vllm_amd.engine.model_runner import ModelRunner
        from byox_vllm_amd.engine.scheduler import Scheduler
        self.config = engine_config(cfg_json, weights, dtype, blocks=blocks, slots=slots, block_size=block_size)
        self.runner = ModelRunner(self.config, 0, None)
        self.scheduler = Scheduler(self.config)
        self.block_size = block_size

    def replay(self, requests: dict, schedule: list):
        """requests: name -> token list; schedule: steps of [(name, count)].  Logits of every position, per request.
        A request ends (and gives back pages and slot) with the step that brings its last token."""
        from byox_vllm_amd.engine.sequence import Sequence
        live, at, out = {}, {n: 0 for n in requests}, {n: [] for n in requests}
        for step in schedule:
            plan = []
            for name, count in step:
                piece = requests[name][at[name]: at[name] + count]
                if name not in live:
                    live[name] = Sequence(piece, self.block_size)
                    self.scheduler.add(live[name])
                else:
                    live[name].extend_tokens(piece)
                plan.append((live[name], count))
                at[name] += count
            self.scheduler.commit(plan)
            logits = self.runner.run_portions(plan, want=[list(range(c)) for _, c in plan]).cpu()
            self.scheduler.advance(plan, [None] * len(plan))
            row = 0
            for name, count in step:
                out[name].append(logits[row: row + count])
                row += count
                if at[name] == len(requests[name]):
                    self.scheduler.finish(live.pop(name))
        return {n: torch.cat(v) for n, v in out.items()}


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per-row error: difference with its mean taken off, root mean square over the vocabulary, relative to the root
    mean square of the expected logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    scale = want.double().pow(2).mean().sqrt()
    return d.pow(2).mean(-1).sqrt() / scale


def row_error(got: torch.Tensor, want: torch.Tensor) -> float:
    return float(row_errors(got, want).max())
