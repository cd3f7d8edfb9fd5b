"""Plain, slow restatement of the Kikelorn design in float64 PyTorch on the CPU: one function per mechanism, whole
sequences only, no cache, no batching, nothing shared with byox_vllm_amd.  Tests compare the engine (portions, pages,
state slots, mixed batches) with these functions run on each request's full token list.

Weights are a dict keyed by the checkpoint's tensor names; ``cfg`` is the config.json dict."""

import math

import torch

F = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rms(x, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def causal_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j), zeros before the first row."""
    T, taps = x.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x])
    return sum(w[:, j] * padded[j:j + T] for j in range(taps))


def rotate(x, positions, freq, magnitude, dims, interleaved):
    """x [T, H, D]: the first ``dims`` numbers of every head are rotated by the angle position * freq[i]; pairs are
    (2i, 2i + 1) when ``interleaved``, else (i, i + dims/2).  Cosine and sine are multiplied by ``magnitude``."""
    a = positions.to(F)[:, None, None] * freq[None, None, :]
    cos, sin = torch.cos(a) * magnitude, torch.sin(a) * magnitude
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = u * cos - v * sin, v * cos + u * sin
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half], out[..., half:dims] = u * cos - v * sin, v * cos + u * sin
    return out


def frequencies(rot):
    """rot = {"base", "dims", "scaling": {"factor", "original", "fast", "slow"} | absent} -> (freq [dims/2], magnitude)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def where(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(sc["fast"]))), 0)
    hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def softmax_attention(q, k, v, scale, visible):
    """q [T, H, d], k [T, G, d], v [T, G, dv], visible [T, T] bool (row: query, column: key) -> [T, H, dv]."""
    H, G = q.shape[1], k.shape[1]
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~visible[None], float("-inf"))
    return torch.einsum("hij,jhv->ihv", torch.softmax(s, -1), v)


def causal(T):
    i = torch.arange(T)
    return i[None, :] <= i[:, None]


def chunked(T, size):
    i = torch.arange(T)
    return causal(T) & ((i[None, :] // size) == (i[:, None] // size))


def attention_mixer(h, W, p, m, eps, shared):
    """Grouped softmax attention inside chunks of the sequence, with a short convolution behind each projection, one
    RMS norm across all heads for q and for k, a partial rotation, values blended with those of the first layer that
    shares them, and one sigmoid gate per head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if m.get("conv"):
        q, k, v = causal_conv(q, W[p + "q.conv"]), causal_conv(k, W[p + "k.conv"]), causal_conv(v, W[p + "v.conv"])
    q, k = rms(q, eps) * W[p + "q.norm"], rms(k, eps) * W[p + "k.norm"]
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    rot = m.get("rot")
    if rot:
        f, mag = frequencies(rot)
        pos = torch.arange(T)
        q, k = rotate(q, pos, f, mag, int(rot["dims"]), False), rotate(k, pos, f, mag, int(rot["dims"]), False)
    if m.get("v_mix"):          # blended as flat rows of G * dv numbers: the layers may cut them into heads differently
        if "v_first" in shared:
            lam = W[p + "vmix"]
            v = ((1.0 - lam) * v.reshape(T, G * dv) + lam * shared["v_first"]).view(T, G, dv)
        else:
            shared["v_first"] = v.reshape(T, G * dv)
    size = (m.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, float(m["scale"]), chunked(T, int(size)) if size else causal(T))
    o = o * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T


def latent_attention_mixer(h, W, p, m, eps, shared):
    """Keys and values of every head are up-projections of one normed low-rank latent per token; one rotated key part is
    shared by the heads; queries go through a latent of their own; the gate has one number per output channel."""
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).view(T, H, d + r)
    down = h @ W[p + "dkv"].T
    c = rms(down[:, :R], eps) * W[p + "dkv.norm"]
    k_rot = down[:, R:].view(T, 1, r)
    rot = dict(m.get("rot") or {"base": 10000.0}, dims=r)
    f, mag = frequencies(rot)
    pos = torch.arange(T)
    q_rot = rotate(q[..., d:], pos, f, mag, r, True)
    k_rot = rotate(k_rot, pos, f, mag, r, True)
    k = torch.cat([(c @ W[p + "uk"].T).view(T, H, d), k_rot.expand(T, H, r)], -1)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    o = softmax_attention(torch.cat([q[..., :d], q_rot], -1), k, v, float(m["scale"]), causal(T))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def min_gru(z, u):
    """z, u [T, C]: S_t = (1 - z_t) S_(t-1) + z_t c_t from S = 0, with c = u + 1/2 for u >= 0 and sigmoid(u) below."""
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(z.shape[1], dtype=F)
    out = []
    for t in range(z.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        out.append(S)
    return torch.stack(out)


def mingru_mixer(h, W, p, m, eps, shared):
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    return (min_gru(z, u) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def feed_forward(h, W, p):
    return gelu_tanh(h @ W[p + "up"].T + W[p + "up.b"]) @ W[p + "down"].T + W[p + "down.b"]


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer, "mingru": mingru_mixer}


def sublayer(x, f, W, canon, rg, norm, taps, eps, mult):
    """x <- x + mult * norm(f(x + conv(x)) * sigmoid(W_rg x + b)): the sublayer reads the residual through a short
    convolution, its result is gated by the residual itself, normed, and added."""
    y = f(x + causal_conv(x, W[canon]) if taps else x)
    y = y * torch.sigmoid(x @ W[rg].T + W[rg + ".b"])
    return x + mult * rms(y, eps) * W[norm]


def forward(tokens, W, cfg, trace=None):
    """Token ids -> logits [T, vocab] (float64).  ``trace`` collects the residual after every layer."""
    W = {k: v.to(F) for k, v in W.items()}
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    taps = int((cfg.get("canon") or {}).get("taps", 0))          # 0: the sublayers read the residual itself
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    shared = {}
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        mixer = MIXERS[spec["type"]]
        x = sublayer(x, lambda h: mixer(h, W, p + "mix.", spec["mixer"], eps, shared), W, p + "canon1", p + "rg1",
                     p + "norm1", taps, eps, mult)
        if spec.get("mlp"):
            x = sublayer(x, lambda h: feed_forward(h, W, p + "mlp."), W, p + "canon2", p + "rg2", p + "norm2", taps,
                         eps, mult)
        if trace is not None:
            trace.append(x)
    return (rms(x, eps) * W["final.norm"]) @ W["embed"].T


def random_weights(cfg, seed=0):
    """A checkpoint of the design's tensor names for ``cfg``, values representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    width, W = cfg["width"], {}
    taps = int((cfg.get("canon") or {}).get("taps", 0))

    def mat(n, k, s=None):
        s = (k ** -0.5) if s is None else s
        return (torch.randn(n, k, generator=g) * s).to(torch.bfloat16)

    def vec(n, s=0.1, at=0.0):
        return (at + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    W["embed"] = mat(cfg["vocab"], width, 1.0)
    for i, spec in enumerate(cfg["layers"]):
        m, p = spec["mixer"], f"l{i}."
        subs = ("1", "2") if spec.get("mlp") else ("1",)
        for s in subs:
            W[p + "norm" + s] = vec(width, 0.2, 1.0)
            W[p + "rg" + s], W[p + "rg" + s + ".b"] = mat(width, width), vec(width, 0.5)
            if taps:
                W[p + "canon" + s] = mat(width, taps, 0.4)
        if spec["type"] == "attention":
            H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
            for name, n in (("q", H * d), ("k", G * d), ("v", G * dv)):
                W[p + "mix." + name] = mat(n, width)
                if m.get("conv"):
                    W[p + "mix." + name + ".conv"] = mat(n, m["conv"], 0.6)
            W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(H * d, 0.3, 1.5), vec(G * d, 0.3, 1.5)
            if m.get("v_mix"):
                W[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.6 + 0.2).to(torch.bfloat16)
            W[p + "mix.g"] = mat(H, width)
            W[p + "mix.o"] = mat(width, H * dv)
        elif spec["type"] == "latent_attention":
            H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            W[p + "mix.dq"], W[p + "mix.dq.norm"] = mat(m["q_rank"], width), vec(m["q_rank"], 0.2, 1.0)
            W[p + "mix.uq"] = mat(H * (d + r), m["q_rank"], 1.5 * m["q_rank"] ** -0.5)
            W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = mat(m["kv_rank"] + r, width), vec(m["kv_rank"], 0.2, 1.0)
            W[p + "mix.uk"] = mat(H * d, m["kv_rank"], 1.5 * m["kv_rank"] ** -0.5)
            W[p + "mix.uv"] = mat(H * dv, m["kv_rank"])
            W[p + "mix.g"] = mat(H * dv, width)
            W[p + "mix.o"] = mat(width, H * dv)
        else:
            C = m["width"]
            W[p + "mix.z"], W[p + "mix.z.b"] = mat(C, width, 2.0 * width ** -0.5), vec(C, 1.0)
            W[p + "mix.x"], W[p + "mix.x.b"] = mat(C, width), vec(C, 0.5)
            W[p + "mix.g"] = mat(C, width)
            W[p + "mix.o"] = mat(width, C)
        if spec.get("mlp"):
            ff = spec["mlp"]["ff"]
            W[p + "mlp.up"], W[p + "mlp.up.b"] = mat(ff, width), vec(ff, 0.3)
            W[p + "mlp.down"], W[p + "mlp.down.b"] = mat(width, ff), vec(width, 0.3)
    W["final.norm"] = vec(width, 0.2, 1.0)
    return W
