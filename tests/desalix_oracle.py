"""Slow float64 oracle for the Desalix decoder.

Written from the equations, one function per mechanism, one whole sequence at
a time, no caches, no batching. It shares no code with kserve_amd: it reads a
config dict (the keys of config.json) and a dict of tensors named like the
checkpoint, and returns what the engine should reproduce.

Desalix in short: a scaled embedding; layers listed one by one, a span of
which is run several times with shared weights (each pass re-injects the
embedding output and adds a per-pass vector); every sublayer is wrapped in
two scalar-gain RMS norms and a per-channel layer scale; the mixer is
chunk-local causal attention with per-head q/k norm, partial rotation, unit
norm values that are themselves rotated (and the head outputs rotated back),
and a per-head sink in the softmax denominator; the feed-forward is a
sigmoid-routed mixture of clamped gated experts whose routing weight scales
the expert's input, plus an always-on shared expert.
"""

import math

import torch

F64 = torch.float64


# ---------------------------------------------------------------- helpers
def attn_cfg(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.3, chunk=8,
             rot_dims=8, rot_base=100.0):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale,
                mask=dict(size=chunk), rot=dict(base=rot_base, dims=rot_dims))


def moe_cfg(experts=4, top=2, ff=12, limit=0.9, shared_ff=20, shared_limit=1.1):
    return dict(
        kind="moe", expert=dict(ff=ff, limit=limit),
        router=dict(experts=experts, top=top),
        shared=dict(ff=shared_ff, limit=shared_limit),
    )


def attn_layer(mlp="default", **kw):
    return {"type": "attention", "mixer": attn_cfg(**kw),
            "mlp": moe_cfg() if mlp == "default" else mlp}


def make_config(vocab=61, width=24, eps=1e-5, emb_scale=0.7, layers=None,
                loop=(1, 2, 2)):
    return {
        "architecture": "Desalix",
        "vocab": vocab,
        "width": width,
        "norm": {"eps": eps},
        "embedding": {"scale": emb_scale},
        "layers": layers if layers is not None else [attn_layer(), attn_layer()],
        "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]},
    }


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Random checkpoint for ``cfg``; values rounded to ``dtype`` so the
    engine and the oracle see identical numbers."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    sd = {}

    def mat(o, i, s=None):
        return torch.randn(o, i, generator=g) * (s if s is not None else i ** -0.5)

    def glu(p, ff):
        sd[p + "gate"] = mat(ff, W, 1.5 * W ** -0.5)
        sd[p + "up"] = mat(ff, W, 1.5 * W ** -0.5)
        sd[p + "down"] = mat(W, ff)

    sd["embed"] = torch.randn(cfg["vocab"], W, generator=g)
    sd["head"] = mat(cfg["vocab"], W)
    sd["final.norm"] = 1.0 + 0.2 * torch.randn((), generator=g)
    sd["loop.step"] = 0.3 * torch.randn(cfg["loop"]["times"], W, generator=g)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ("norm1", "norm2", "norm1b", "norm2b"):
            sd[p + n] = 1.0 + 0.2 * torch.randn((), generator=g)
        sd[p + "ls1"] = 0.5 + 0.2 * torch.randn(W, generator=g)
        sd[p + "ls2"] = 0.5 + 0.2 * torch.randn(W, generator=g)
        m = layer["mixer"]
        sd[p + "mix.q"] = mat(m["heads"] * m["dim"], W)
        sd[p + "mix.k"] = mat(m["kv_heads"] * m["dim"], W)
        sd[p + "mix.v"] = mat(m["kv_heads"] * m["vdim"], W)
        sd[p + "mix.q.norm"] = 1.0 + 0.3 * torch.randn(m["dim"], generator=g)
        sd[p + "mix.k.norm"] = 1.0 + 0.3 * torch.randn(m["dim"], generator=g)
        sd[p + "mix.sink"] = torch.randn(m["heads"], generator=g)
        sd[p + "mix.o"] = mat(W, m["heads"] * m["vdim"])
        f = layer["mlp"]
        if f is not None:
            for e in range(f["router"]["experts"]):
                glu(p + f"mlp.e{e}.", f["expert"]["ff"])
            sd[p + "mlp.router"] = mat(f["router"]["experts"], W, 2.0 * W ** -0.5)
            if f.get("shared"):
                glu(p + "mlp.shared.", f["shared"]["ff"])
    return {k: v.to(dtype) for k, v in sd.items()}


# ------------------------------------------------------------- mechanisms
def rms_unit(x, eps):
    """x divided by its root mean square over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, gain, eps):
    return rms_unit(x, eps) * gain.to(F64)


def rotate_halves(x, positions, n_rot, base, sign=1.0):
    """Rotate the first ``n_rot`` coordinates of the last axis: coordinate i
    pairs with i + n_rot/2, pair i turns by sign * p * base^(-2i/n_rot).
    x [T, heads, D], positions [T]."""
    half = n_rot // 2
    i = torch.arange(half, dtype=F64)
    freq = base ** (-2.0 * i / n_rot)
    a = sign * positions.to(F64)[:, None, None] * freq
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:n_rot]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., n_rot:]], dim=-1)


def chunk_visible(T, size, offset=0):
    """[T, T] bool: query i sees key j iff j <= i and both lie in the same
    block of ``size`` positions counted from position 0."""
    p = torch.arange(offset, offset + T)
    same = (p[:, None] // size) == (p[None, :] // size)
    return same & (p[None, :] <= p[:, None])


def sink_softmax(scores, visible, sink):
    """Softmax over visible keys whose denominator also holds exp(sink).
    scores [H, T, T], visible [T, T], sink [H]."""
    s = scores.masked_fill(~visible, -math.inf)
    m = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - m))


def attention(h, sd, p, m, eps):
    """h [T, W] -> [T, W]."""
    T = h.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ sd[p + "q"].to(F64).T).view(T, H, D)
    k = (h @ sd[p + "k"].to(F64).T).view(T, G, D)
    v = (h @ sd[p + "v"].to(F64).T).view(T, G, DV)
    q = rms_unit(q, eps) * sd[p + "q.norm"].to(F64)
    k = rms_unit(k, eps) * sd[p + "k.norm"].to(F64)
    base, n_rot = m["rot"]["base"], m["rot"]["dims"]
    q = rotate_halves(q, pos, n_rot, base)
    k = rotate_halves(k, pos, n_rot, base)
    v = rotate_halves(rms_unit(v, eps), pos, DV, base)
    rep = H // G
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    w = sink_softmax(scores, chunk_visible(T, m["mask"]["size"]),
                     sd[p + "sink"].to(F64))
    o = torch.einsum("hij,jhd->ihd", w, v)
    o = rotate_halves(o, pos, DV, base, sign=-1.0)
    return o.reshape(T, H * DV) @ sd[p + "o"].to(F64).T


def clamped_expert(h, sd, p, limit):
    g = torch.clamp(h @ sd[p + "gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ sd[p + "up"].to(F64).T, -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ sd[p + "down"].to(F64).T


def route(h, router_w, top):
    """Returns (indices [T, top], weights [T, top]): the largest sigmoid
    scores, used as they are."""
    s = torch.sigmoid(h @ router_w.to(F64).T)
    w, idx = s.topk(top, dim=-1)
    return idx, w


def moe(h, sd, p, f):
    idx, w = route(h, sd[p + "router"], f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            out[t] += clamped_expert(
                (we * h[t])[None], sd, p + f"e{e}.", f["expert"]["limit"]
            )[0]
    if f.get("shared"):
        out = out + clamped_expert(h, sd, p + "shared.", f["shared"]["limit"])
    return out


def layer_forward(x, sd, i, layer, eps):
    p = f"l{i}."
    h = scalar_norm(x, sd[p + "norm1"], eps)
    d = attention(h, sd, p + "mix.", layer["mixer"], eps)
    x = x + scalar_norm(d, sd[p + "norm1b"], eps) * sd[p + "ls1"].to(F64)
    if layer["mlp"] is not None:
        h = scalar_norm(x, sd[p + "norm2"], eps)
        d = moe(h, sd, p + "mlp.", layer["mlp"])
        x = x + scalar_norm(d, sd[p + "norm2b"], eps) * sd[p + "ls2"].to(F64)
    return x


def layer_runs(cfg):
    """[(layer index, pass number or None)] in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = lp["start"], lp["stop"], lp["times"]
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t) for i in range(a, b)]
    runs += [(i, None) for i in range(b, n)]
    return runs


def forward(cfg, sd, tokens, return_residuals=False):
    """Logits [T, vocab] (float64) of one whole sequence."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    emb = sd["embed"].to(F64)[tokens] * cfg["embedding"]["scale"]
    x = emb.clone()
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    residuals = []
    for i, t in layer_runs(cfg):
        if t is not None and i == lp["start"]:
            if t > 0:
                x = x + emb
            x = x + sd["loop.step"].to(F64)[t]
        x = layer_forward(x, sd, i, cfg["layers"][i], eps)
        residuals.append(x.clone())
    logits = scalar_norm(x, sd["final.norm"], eps) @ sd["head"].to(F64).T
    if return_residuals:
        return logits, residuals
    return logits
