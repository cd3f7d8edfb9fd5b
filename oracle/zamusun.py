"""Plain, slow restatement of the Zamusun design in float64 PyTorch on the CPU: one function per mechanism, whole
sequences only, no cache, no batching, nothing shared with byox_vllm_amd.  Tests compare the engine (portions, pages,
state slots, mixed batches) with these functions run on each request's full token list.

Weights are a dict keyed by the checkpoint's tensor names; ``cfg`` is the config.json dict."""

import math

import torch

F = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def rms(x, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose stored weight sits around zero."""
    return rms(x, eps) * (1.0 + w)


def lightning(q, k, v, decay):
    """q, k [T, H, d], v [T, H, dv] (already activated), decay [H]: S <- decay S + k v^T, o = S^T q.  -> [T, H, dv]"""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=F)
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out)


def lightning_mixer(h, W, pre, m, eps):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ W[pre + "q"].T).view(T, H, d)
    k = silu(h @ W[pre + "k"].T).view(T, H, d)
    v = silu(h @ W[pre + "v"].T).view(T, H, dv)
    o = lightning(q, k, v, torch.tensor(m["decay"], dtype=F)).reshape(T, H * dv)
    o = rms(o, eps) * W[pre + "norm"] * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def soft_bound(z, cap):
    return cap * torch.tanh(z / cap)


def mlstm(q, k, v, i_log, f_log):
    """Matrix memory with a running maximum that starts at 0.  q (already scaled), k [T, H, d], v [T, H, dv], log gates
    [T, H].  -> [T, H, dv]"""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=F)
    n = torch.zeros(H, d, dtype=F)
    m = torch.zeros(H, dtype=F)
    out = []
    for t in range(T):
        m_new = torch.maximum(f_log[t] + m, i_log[t])
        keep, take = torch.exp(f_log[t] + m - m_new), torch.exp(i_log[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out.append(num / den[:, None])
    return torch.stack(out)


def mlstm_mixer(h, W, pre, m, eps):
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    T = h.shape[0]
    q = (h @ W[pre + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[pre + "k"].T).view(T, H, d)
    v = (h @ W[pre + "v"].T).view(T, H, dv)
    i_log = soft_bound(h @ W[pre + "i"].T + W[pre + "i.b"], cap)
    f_log = torch.nn.functional.logsigmoid(soft_bound(h @ W[pre + "f"].T + W[pre + "f.b"], cap))
    o = rms(mlstm(q, k, v, i_log, f_log), eps).reshape(T, H * dv)
    o = o * W[pre + "norm"] * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def query_temperature(T, coef, every):
    p = torch.arange(T, dtype=F)
    return 1.0 + coef * torch.log(torch.floor((p + 1.0) / every) + 1.0)


def sink_attention(q, k, scale, sink):
    """Causal softmax attention whose values are the keys and whose denominator also holds exp(sink) per query head.
    q [T, H, d], k [T, G, d], sink [H].  -> [T, H, d]"""
    T, H, d = q.shape
    G = k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)                        # query head h reads key head h // (H / G)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
    top = torch.maximum(s.max(-1).values, sink[:, None])
    e = torch.exp(s - top[..., None])
    den = e.sum(-1) + torch.exp(sink[:, None] - top)
    return torch.einsum("hij,jhd->ihd", e / den[..., None], kk)


def attention_mixer(h, W, pre, m, eps):
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = (h @ W[pre + "q"].T + W[pre + "q.b"]).view(T, H, d)
    k = (h @ W[pre + "k"].T + W[pre + "k.b"]).view(T, G, d)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, float(qt["coef"]), int(qt["every"]))[:, None, None]
    o = sink_attention(q, k, float(m["scale"]), W[pre + "sink"]).reshape(T, H * d)
    o = o * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T + W[pre + "o.b"]


def route(z, top):
    """Router logits [T, E] -> (chosen experts [T, top], their softmax scores divided by their sum)."""
    s = torch.softmax(z, -1)
    val, idx = s.topk(top, dim=-1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20)


def expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def moe(h, W, pre, spec):
    E, top, limit = spec["router"]["experts"], spec["router"]["top"], float(spec["expert"]["limit"])
    idx, wt = route(h @ W[pre + "router"].T, top)
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += wt[t, j] * expert(h[t], W[f"{pre}e{e}.gate"], W[f"{pre}e{e}.up"], W[f"{pre}e{e}.down"], limit)
    return out


MIXERS = {"lightning": lightning_mixer, "mlstm": mlstm_mixer, "attention": attention_mixer}


def layer_runs(cfg):
    """Order in which the layers run: (layer index, first of a repeated pass?) with the looped span repeated."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(tokens, W, cfg, trace=None):
    """Token ids -> logits [T, vocab] (float64).  ``trace`` collects the residual after every layer run."""
    W = {k: v.to(F) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x0 = x
    for i, enters_pass in layer_runs(cfg):
        spec = cfg["layers"][i]
        if enters_pass:
            x = torch.cat([x, x0], -1) @ W["loop.in"].T
        h = norm_one_plus(x, W[f"l{i}.norm1"], eps)
        y = MIXERS[spec["type"]](h, W, f"l{i}.mix.", spec["mixer"], eps)
        if spec.get("mlp"):
            y = y + moe(h, W, f"l{i}.mlp.", spec["mlp"])
        x = x + y
        if trace is not None:
            trace.append(x)
    return norm_one_plus(x, W["final.norm"], eps) @ W["embed"].T


def random_weights(cfg, seed=0, scale=None):
    """A checkpoint of the design's tensor names for ``cfg``, values representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    width, W = cfg["width"], {}

    def mat(n, k, s=None):
        s = (k ** -0.5) if s is None else s
        return (torch.randn(n, k, generator=g) * s).to(torch.bfloat16)

    def vec(n, s=0.1, at=0.0):
        return (at + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    W["embed"] = mat(cfg["vocab"], width, 1.0)
    if cfg.get("loop"):
        W["loop.in"] = mat(width, 2 * width, (2 * width) ** -0.5 * 1.4)
    for i, spec in enumerate(cfg["layers"]):
        m, p = spec["mixer"], f"l{i}."
        W[p + "norm1"] = vec(width)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        if spec["type"] == "attention":
            G = m["kv_heads"]
            W[p + "mix.q"], W[p + "mix.q.b"] = mat(H * d, width), vec(H * d)
            W[p + "mix.k"], W[p + "mix.k.b"] = mat(G * d, width), vec(G * d)
            W[p + "mix.sink"] = vec(H, 1.0)
            W[p + "mix.g"] = mat(H * dv, width)
            W[p + "mix.o"], W[p + "mix.o.b"] = mat(width, H * dv), vec(width)
        else:
            for name, n in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                W[p + "mix." + name] = mat(n, width)
            W[p + "mix.o"] = mat(width, H * dv)
            W[p + "mix.norm"] = vec(H * dv, 0.1, 1.0)
            if spec["type"] == "mlstm":
                W[p + "mix.i"], W[p + "mix.i.b"] = mat(H, width), vec(H, 0.5)
                W[p + "mix.f"], W[p + "mix.f.b"] = mat(H, width), vec(H, 0.5, 2.0)
        mlp = spec.get("mlp")
        if mlp:
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"] = mat(ff, width), mat(ff, width)
                W[f"{p}mlp.e{e}.down"] = mat(width, ff)
            W[p + "mlp.router"] = mat(mlp["router"]["experts"], width, 2.0 * width ** -0.5)
    W["final.norm"] = vec(width)
    return W
