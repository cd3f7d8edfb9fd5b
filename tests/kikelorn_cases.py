"""Small Kikelorn configurations, helpers and an engine harness shared by the host and GPU tests.  Sizes are deliberately
awkward: key and value sizes that differ, head counts that are no powers of two, widths that are no multiples of 8,
chunks that are no multiples of a page and one that is a page, one tap and five, a residual multiplier and an embedding
scale of one, a recurrent layer first, a layer without a feed-forward, a rotation over all of a head and over part of it,
latent ranks that do and do not fit the matrix-core kernels, values shared by two layers of different head counts."""

import copy

import torch

from oracle import kikelorn as O


def attention(heads, kv_heads, dim, vdim, scale, chunk=None, taps=None, rot=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        m["mask"] = {"size": chunk}
    if taps:
        m["conv"] = taps
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base=10000.0, scaling=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                                                  "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale, "rot": rot}}


def mingru(width):
    return {"type": "mingru", "mixer": {"width": width}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(vocab, width, layers, taps=2, mult=0.8, scale=1.0, eps=1e-5):
    cfg = {"architecture": "Kikelorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "embedding": {"scale": scale}, "layers": [dict(copy.deepcopy(mixer), mlp=mlp) for mixer, mlp in layers]}
    if taps:
        cfg["canon"] = {"taps": taps}
    return cfg


def mixed_config():
    """A recurrent layer first; two attention layers of different head counts that share values (6 x 8 = 2 x 24); three
    query heads per key head; chunks of 20 and 7 tokens against pages of 16; four input taps; one layer without a
    feed-forward."""
    return config(150, 96, [
        (mingru(80), dense(64)),
        (attention(6, 2, 16, 24, 0.3, chunk=20, taps=3, rot=(500.0, 8), v_mix=True), dense(40)),
        (latent(3, 16, 8, 24, 40, 32, 0.2, base=3000.0, scaling=(8.0, 64, 16.0, 2.0)), None),
        (attention(2, 2, 24, 24, 0.25, chunk=7, taps=2, rot=(100.0, 24), v_mix=True), dense(72)),
        (mingru(50), None),
    ], taps=4, mult=0.7, scale=1.5)


def odd_config():
    """Nothing is a multiple of 8; single heads; one input tap (the convolution is a per-channel factor); multiplier
    and embedding scale of one; an attention layer without chunks, rotation or shared values, five taps behind its
    projections; a latent rank that leaves the matrix-core kernel out; no frequency scaling."""
    return config(77, 100, [
        (latent(1, 12, 4, 20, 12, 20, 0.4), dense(36)),
        (attention(1, 1, 20, 12, 0.3, taps=5), None),
        (mingru(36), dense(28)),
    ], taps=1, mult=1.0, scale=1.0, eps=1e-6)


def aligned_config():
    """Sizes in multiples of 16 and 32, where the 16-bit engine takes its matrix-core kernels; a chunk of one page; a
    rotation over half of each head; four query heads per key head; an attention layer without a convolution."""
    return config(256, 128, [
        (attention(8, 2, 32, 32, 32 ** -0.5, chunk=16, taps=4, rot=(10000.0, 16), v_mix=True), dense(96)),
        (latent(4, 32, 16, 32, 48, 64, 48 ** -0.5, base=50000.0, scaling=(4.0, 32, 8.0, 1.0)), dense(128)),
        (mingru(128), dense(64)),
        (attention(4, 4, 64, 16, 0.125, chunk=40, rot=(1000.0, 64), v_mix=True), None),
    ], taps=2, mult=0.6, scale=2.0)


def plain_config():
    """No input convolution at all (no 'canon' entry); one attention layer that shares values with nobody; heads of 128
    with eight query heads on one key head."""
    return config(90, 64, [
        (attention(8, 1, 128, 40, 0.09, chunk=33, taps=4, rot=(20000.0, 32), v_mix=True), dense(48)),
        (mingru(64), None),
        (latent(2, 24, 8, 16, 16, 48, 0.18, scaling=(2.0, 16, 4.0, 1.0)), dense(32)),
    ], taps=0, mult=0.25, scale=1.25)


def random_config(seed: int):
    """A configuration drawn from a seed: three to six layers of any kind in any order, head counts, sizes, chunks, taps,
    ranks and constants drawn independently (sharing layers agree on the size of a token's values, nothing else)."""
    import random
    rng = random.Random(seed)
    width = rng.choice([64, 72, 96, 100, 128, 160, 192])
    shared, layers = None, []
    for _ in range(rng.randint(3, 6)):
        kind = rng.choice(["attention", "latent", "mingru"])
        if kind == "attention":
            G = rng.choice([1, 2, 3, 4])
            H = G * rng.choice([1, 2, 3, 4])
            d, dv = rng.choice([16, 24, 32, 48, 64]), rng.choice([8, 16, 24, 40, 64])
            v_mix = rng.random() < 0.7
            if v_mix and shared is None:
                shared = (G, dv)
            elif v_mix:
                (G, dv), H = shared, shared[0] * rng.choice([1, 2, 4])
            rot = rng.choice([0, 2, d // 2, d]) // 2 * 2
            mixer = attention(H, G, d, dv, rng.choice([d ** -0.5, 0.1, 0.3]), chunk=rng.choice([None, 5, 16, 33, 64, 100]),
                              taps=rng.choice([None, 2, 3, 5]), rot=(rng.choice([100.0, 1e4, 1e6]), rot) if rot else None,
                              v_mix=v_mix)
        elif kind == "latent":
            d, r = rng.choice([8, 16, 24, 32, 64]), rng.choice([2, 4, 8, 16, 32])
            scaling = (rng.choice([2.0, 4.0, 8.0]), rng.choice([16, 64, 1024]), rng.choice([8.0, 32.0]),
                       rng.choice([1.0, 2.0])) if rng.random() < 0.7 else None
            mixer = latent(rng.choice([1, 2, 3, 4, 8]), d, r, rng.choice([8, 16, 24, 32, 64]), rng.choice([12, 16, 32]),
                           rng.choice([16, 20, 32, 48, 64]), rng.choice([(d + r) ** -0.5, 0.15]),
                           base=rng.choice([1e3, 1e4, 1e6]), scaling=scaling)
        else:
            mixer = mingru(rng.choice([8, 36, 64, 100, 200]))
        layers.append((mixer, dense(rng.choice([16, 40, 64, 128])) if rng.random() < 0.8 else None))
    return config(rng.choice([97, 256, 300]), width, layers, taps=rng.choice([0, 1, 2, 3, 4, 5]),
                  mult=rng.choice([0.25, 0.5, 1.0]), scale=rng.choice([1.0, 2.0, 4.0]), eps=rng.choice([1e-5, 1e-6]))


def random_checkpoint(cfg, seed=0):
    return O.random_weights(cfg, seed)


def engine_config(cfg_json, weights, dtype, blocks=16, slots=4, block_size=16, **kw):
    """The engine's Config for an in-memory checkpoint of one of the configurations above."""
    from byox_vllm_amd.config import Config
    from byox_vllm_amd.models.kikelorn import kikelorn_config
    hf = kikelorn_config(cfg_json, dtype=dtype)
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
