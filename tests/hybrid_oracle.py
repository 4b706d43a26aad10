"""Slow float64 oracle for the per-layer hybrid decoder (Merulorn design).

Written from the equations, one function per mechanism, whole sequences at a
time, no caches, no batching. It shares no code with kserve_amd: it reads a
config dict (the keys of config.json) and a dict of tensors named like the
checkpoint, and returns what the engine should reproduce.
"""

import math

import torch

F64 = torch.float64


# ---------------------------------------------------------------- helpers
def make_config(
    vocab=97, width=48, eps=1e-5, emb_scale=3.0, layers=None,
):
    return {
        "architecture": "Merulorn",
        "vocab": vocab,
        "width": width,
        "norm": {"eps": eps},
        "embedding": {"scale": emb_scale},
        "layers": layers,
    }


def ssm_cfg(heads=4, vdim=8, state=16, groups=2, conv=4, norm_groups=2):
    return dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv,
                norm_groups=norm_groups)


def attn_cfg(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.3, coef=0.7, every=5):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale,
                q_temp=dict(coef=coef, every=every))


def mamba_layer(mlp=None, **kw):
    return {"type": "mamba2", "mixer": ssm_cfg(**kw), "mlp": mlp}


def parallel_layer(left=None, right=None, left_scale=0.8, right_scale=1.3, mlp=None):
    return {
        "type": "parallel",
        "mixer": {
            "left": left or attn_cfg(),
            "right": right or ssm_cfg(),
            "left_scale": left_scale,
            "right_scale": right_scale,
        },
        "mlp": mlp,
    }


def dense_mlp(ff=40, limit=0.9):
    return {"kind": "dense", "ff": ff, "limit": limit}


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Random checkpoint for ``cfg``; values rounded to ``dtype`` so the
    engine and the oracle see identical numbers."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    sd = {}

    def mat(o, i, s=None):
        return torch.randn(o, i, generator=g) * (s if s is not None else i ** -0.5)

    def vec(n, s=0.1):
        return torch.randn(n, generator=g) * s

    def ssm(p, m):
        inner = m["heads"] * m["vdim"]
        ch = inner + 2 * m["groups"] * m["state"]
        sd[p + "in"] = mat(2 * inner + 2 * m["groups"] * m["state"] + m["heads"], W)
        sd[p + "conv"] = torch.randn(ch, m["conv"], generator=g) * 0.5
        sd[p + "conv.b"] = vec(ch)
        sd[p + "dt_bias"] = torch.rand(m["heads"], generator=g) * 2 - 2
        sd[p + "A_log"] = torch.rand(m["heads"], generator=g) * 2 - 1
        sd[p + "D"] = vec(m["heads"], 1.0)
        sd[p + "norm"] = 1 + vec(inner)
        sd[p + "o"] = mat(W, inner)

    def attn(p, m):
        sd[p + "q"] = mat(m["heads"] * m["dim"], W)
        sd[p + "k"] = mat(m["kv_heads"] * m["dim"], W)
        sd[p + "v"] = mat(m["kv_heads"] * m["vdim"], W)
        for n, rows in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]),
                        ("v", m["kv_heads"] * m["vdim"])):
            sd[p + n + ".b"] = vec(rows)
        sd[p + "q.norm"] = 1 + vec(m["heads"] * m["dim"])
        sd[p + "k.norm"] = 1 + vec(m["kv_heads"] * m["dim"])
        sd[p + "g"] = mat(m["heads"], W)
        sd[p + "o"] = mat(W, m["heads"] * m["vdim"])

    sd["embed"] = torch.randn(cfg["vocab"], W, generator=g) * 0.3
    sd["head"] = mat(cfg["vocab"], W)
    sd["final.norm"] = vec(W)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        sd[p + "norm1"] = vec(W)
        if L["type"] == "mamba2":
            ssm(p + "mix.", L["mixer"])
        else:
            attn(p + "mix.left.", L["mixer"]["left"])
            ssm(p + "mix.right.", L["mixer"]["right"])
        if L["mlp"]:
            sd[p + "norm2"] = vec(W)
            sd[p + "mlp.gate"] = mat(L["mlp"]["ff"], W, 1.5 * W ** -0.5)
            sd[p + "mlp.up"] = mat(L["mlp"]["ff"], W, 1.5 * W ** -0.5)
            sd[p + "mlp.down"] = mat(W, L["mlp"]["ff"])
    return {k: v.to(dtype).float() for k, v in sd.items()}


# ------------------------------------------------------------- mechanisms
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight sits around zero."""
    return rms(x, eps) * (1.0 + w)


def embed(tokens, table, scale):
    n, width = len(tokens), table.shape[1]
    x = table[tokens].to(F64) * scale
    for p in range(n):
        for i in range(width):
            ang = p * 10000.0 ** (-(2 * (i // 2)) / width)
            x[p, i] += math.cos(ang) if i % 2 else math.sin(ang)
    return x


def causal_conv(u, w, b):
    """u [T, C]; w [C, taps], last column multiplies the current token."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = b.clone()
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                acc = acc + w[:, j] * u[src]
        out[t] = acc
    return out


def silu(x):
    return x / (1.0 + torch.exp(-x))


def softplus(x):
    return torch.log1p(torch.exp(x))


def ssd(x, B, C, dt, a_log, d_skip, groups):
    """x [T, H, P], B/C [T, G, N], dt [T, H] (already positive)."""
    T, H, P = x.shape
    N = B.shape[2]
    y = torch.zeros(T, H, P, dtype=F64)
    for h in range(H):
        g = h // (H // groups)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = math.exp(-math.exp(a_log[h]) * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + d_skip[h] * x[t, h]
    return y


def ssm_mixer(h, sd, p, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ sd[p + "in"].to(F64).T
    z = proj[:, :inner]
    u = proj[:, inner : 2 * inner + 2 * G * N]
    dt = softplus(proj[:, 2 * inner + 2 * G * N :] + sd[p + "dt_bias"].to(F64))
    u = silu(causal_conv(u, sd[p + "conv"].to(F64), sd[p + "conv.b"].to(F64)))
    x = u[:, :inner].reshape(T, H, P)
    B = u[:, inner : inner + G * N].reshape(T, G, N)
    C = u[:, inner + G * N :].reshape(T, G, N)
    y = ssd(x, B, C, dt, sd[p + "A_log"].to(F64), sd[p + "D"].to(F64), G).reshape(T, inner)
    y = y * silu(z)
    parts = y.reshape(T, m["norm_groups"], -1)
    y = rms(parts, eps).reshape(T, inner) * sd[p + "norm"].to(F64)
    return y @ sd[p + "o"].to(F64).T


def attention_mixer(h, sd, p, m, eps):
    T = h.shape[0]
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ sd[p + "q"].to(F64).T + sd[p + "q.b"].to(F64)
    k = h @ sd[p + "k"].to(F64).T + sd[p + "k.b"].to(F64)
    v = h @ sd[p + "v"].to(F64).T + sd[p + "v.b"].to(F64)
    q = rms(q, eps) * sd[p + "q.norm"].to(F64)
    k = rms(k, eps) * sd[p + "k.norm"].to(F64)
    qt = m.get("q_temp")
    for t in range(T):
        if qt:
            q[t] = q[t] * (1.0 + qt["coef"] * math.log((t + 1) // qt["every"] + 1))
    gate = 1.0 / (1.0 + torch.exp(-(h @ sd[p + "g"].to(F64).T)))
    out = torch.zeros(T, H * DV, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            sc = (k[: t + 1, g * D : (g + 1) * D] @ q[t, hd * D : (hd + 1) * D]) * m["scale"]
            wgt = torch.softmax(sc, 0)
            out[t, hd * DV : (hd + 1) * DV] = (wgt @ v[: t + 1, g * DV : (g + 1) * DV]) * gate[t, hd]
    return out @ sd[p + "o"].to(F64).T


def glu(h, sd, p, m):
    lim = m["limit"]
    g = torch.clamp(h @ sd[p + "gate"].to(F64).T, max=lim)
    u = torch.clamp(h @ sd[p + "up"].to(F64).T, -lim, lim)
    return (g / (1.0 + torch.exp(-1.702 * g)) * (u + 1.0)) @ sd[p + "down"].to(F64).T


def forward(cfg, sd, tokens, residuals=None):
    """Logits [T, vocab] (float64) of one whole sequence."""
    eps = cfg["norm"]["eps"]
    x = embed(tokens, sd["embed"], cfg["embedding"]["scale"])
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_norm(x, sd[p + "norm1"].to(F64), eps)
        if L["type"] == "mamba2":
            x = x + ssm_mixer(h, sd, p + "mix.", L["mixer"], eps)
        else:
            m = L["mixer"]
            x = (
                x
                + m["left_scale"] * attention_mixer(h, sd, p + "mix.left.", m["left"], eps)
                + m["right_scale"] * ssm_mixer(h, sd, p + "mix.right.", m["right"], eps)
            )
        if L["mlp"]:
            x = x + glu(offset_norm(x, sd[p + "norm2"].to(F64), eps), sd, p + "mlp.", L["mlp"])
        if residuals is not None:
            residuals.append(x.clone())
    return offset_norm(x, sd["final.norm"].to(F64), eps) @ sd["head"].to(F64).T
