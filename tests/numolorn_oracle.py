"""A plain, slow formulation of the Numolorn design's mechanisms, one function
per mechanism, written from its equations for whole sequences (no cache, no
batching, no steps). float64 throughout; it shares no code with the serving
path and is what the tests compare against.

Weights arrive as a dict of tensors under their checkpoint names
('l<i>.mix.q', 'l<i>.mlp.e<j>.up', ...), linear weights stored [out, in].
"""

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def lin(w, x):
    return x @ w.to(F64).t()


# ------------------------------------------------------------- embedding
def embedding(tokens, w, cfg):
    """Token row plus a hashed row for the pair (previous, current); the
    first token of a sequence takes the table's last row."""
    bg = cfg["embedding"]["bigram"]
    n, a, b = int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])
    rows = []
    for i, t in enumerate(tokens):
        rows.append(n if i == 0 else (tokens[i - 1] * a + t * b) % n)
    ids = torch.tensor(tokens, dtype=torch.long)
    return w["embed"].to(F64)[ids] + \
        w["bigram"].to(F64)[torch.tensor(rows, dtype=torch.long)]


# -------------------------------------------------------------- rotation
def rotate_half(x, dims, base):
    """x [L, heads, d]; coordinate i pairs with i + dims/2 among the first
    ``dims``; position p turns pair i by p * base^(-2i/dims)."""
    L, half = x.shape[0], dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)],
                     dtype=F64)
    ang = torch.arange(L, dtype=F64)[:, None] * f[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ------------------------------------------------------------- attention
def attend(q, k, v, scale, window=None, sink=None):
    """q, k [L, H, d], v [L, H, dv]. Position i sees j <= i, with a window
    only those with i - j < window. ``sink`` [H] joins the softmax's
    denominator as one more (unscaled) logit without a value."""
    L, H = q.shape[0], q.shape[1]
    out = torch.zeros(L, H, v.shape[2], dtype=F64)
    for i in range(L):
        lo = 0 if window is None else max(0, i - window + 1)
        for h in range(H):
            s = (k[lo:i + 1, h] @ q[i, h]) * scale
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            den = e.sum()
            if sink is not None:
                den = den + torch.exp(sink[h] - m)
            out[i, h] = (e[:, None] * v[lo:i + 1, h]).sum(0) / den
    return out


def latent_attention(h, w, pre, m, eps):
    """Queries through a normed latent; keys and values from a normed latent
    plus one rotated key part shared by the heads; sink; per-head gate."""
    L = h.shape[0]
    H, d, r, dv, rank = (int(m[k]) for k in
                         ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    cq = rms(lin(w[pre + "dq"], h), eps) * w[pre + "dq.norm"].to(F64)
    q = lin(w[pre + "uq"], cq).view(L, H, d + r)
    kv = lin(w[pre + "dkv"], h)
    c = rms(kv[:, :rank], eps) * w[pre + "dkv.norm"].to(F64)
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    k_rot = rotate_half(kv[:, rank:].view(L, 1, r), dims, base)
    q_rot = rotate_half(q[..., d:], dims, base)
    k = torch.cat([lin(w[pre + "uk"], c).view(L, H, d),
                   k_rot.expand(L, H, r)], -1)
    v = lin(w[pre + "uv"], c).view(L, H, dv)
    o = attend(torch.cat([q[..., :d], q_rot], -1), k, v, float(m["scale"]),
               sink=w[pre + "sink"].to(F64))
    o = o * sigmoid(lin(w[pre + "g"], h))[:, :, None]
    return lin(w[pre + "o"], o.reshape(L, H * dv))


def latent_window_attention(h, w, pre, m, eps):
    """No positions: keys and values from a normed latent, sliding window."""
    L = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = lin(w[pre + "q"], h).view(L, H, d)
    c = rms(lin(w[pre + "dkv"], h), eps) * w[pre + "dkv.norm"].to(F64)
    k = lin(w[pre + "uk"], c).view(L, H, d)
    v = lin(w[pre + "uv"], c).view(L, H, dv)
    o = attend(q, k, v, float(m["scale"]), window=int(m["mask"]["size"]))
    return lin(w[pre + "o"], o.reshape(L, H * dv))


# ------------------------------------------------------------ recurrence
def causal_conv(x, w):
    """x [L, C]; w [C, taps], the last column multiplies the current input;
    zeros before the start."""
    L, C = x.shape
    taps = w.shape[1]
    w = w.to(F64)
    out = torch.zeros(L, C, dtype=F64)
    for t in range(L):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                out[t] += w[:, j] * x[s]
    return out


def channel_delta(h, w, pre, m, eps):
    """Gated delta rule whose decay differs per head AND key channel."""
    L = h.shape[0]
    H, G, d, dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    q = silu(causal_conv(lin(w[pre + "q"], h), w[pre + "q.conv"])).view(L, G, d)
    k = silu(causal_conv(lin(w[pre + "k"], h), w[pre + "k.conv"])).view(L, G, d)
    v = silu(causal_conv(lin(w[pre + "v"], h), w[pre + "v.conv"])).view(L, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(lin(w[pre + "b"], h))                           # [L, H]
    z = lin(w[pre + "a2"], lin(w[pre + "a1"], h)) + w[pre + "dt_bias"].to(F64)
    rate = torch.exp(w[pre + "A_log"].to(F64))[None, :, None]
    g = torch.exp(-rate * softplus(z).view(L, H, d))               # [L, H, d]
    gate = sigmoid(lin(w[pre + "g2"], lin(w[pre + "g1"], h))).view(L, H, dv)
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(L, H, dv, dtype=F64)
    rep = H // G
    for t in range(L):
        for hh in range(H):
            kk, qq = k[t, hh // rep], q[t, hh // rep]
            S[hh] = g[t, hh][:, None] * S[hh]
            u = beta[t, hh] * (v[t, hh] - S[hh].t() @ kk)
            S[hh] = S[hh] + kk[:, None] * u[None, :]
            o[t, hh] = S[hh].t() @ qq
    o = rms(o, eps) * w[pre + "norm"].to(F64) * gate
    return lin(w[pre + "o"], o.reshape(L, H * dv))


# ---------------------------------------------------------- feed-forward
def dense_ff(h, w, pre):
    return lin(w[pre + "down"], silu(lin(w[pre + "gate"], h))
               * lin(w[pre + "up"], h))


def route(h, w, pre, r):
    """Returns [(expert, weight), ...] per token."""
    E, top = int(r["experts"]), int(r["top"])
    n = E + int(r.get("identity", 0))
    s = torch.softmax(lin(w[pre + "router"], h), -1)               # [L, n]
    c = s + w[pre + "correction"].to(F64)
    gr = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(gr["count"]), int(gr["keep"])
    size = n // count
    picks = []
    for t in range(h.shape[0]):
        best = sorted(range(count), key=lambda j: -float(
            c[t, j * size:(j + 1) * size].max()))[:keep]
        allowed = [e for e in range(n) if e // size in best]
        chosen = sorted(allowed, key=lambda e: -float(c[t, e]))[:top]
        tot = sum(float(s[t, e]) for e in chosen) + 1e-20
        picks.append([(e, float(s[t, e]) / tot * float(r["scale"]))
                      for e in chosen])
    return picks


def expert(h, w, pre, limit):
    g = torch.clamp(lin(w[pre + "gate"], h), max=limit)
    u = torch.clamp(lin(w[pre + "up"], h), -limit, limit)
    return lin(w[pre + "down"], g * sigmoid(1.702 * g) * (u + 1.0))


def moe_ff(h, w, pre, mlp):
    E, limit = int(mlp["router"]["experts"]), float(mlp["expert"]["limit"])
    out = torch.zeros_like(h)
    for t, picks in enumerate(route(h, w, pre, mlp["router"])):
        for e, wt in picks:
            y = h[t] if e >= E else expert(h[t:t + 1], w, f"{pre}e{e}.",
                                           limit)[0]
            out[t] += wt * y
    return out


# ----------------------------------------------------------------- model
MIXERS = {"latent_attention": latent_attention,
          "latent_attention_2": latent_window_attention,
          "channel_delta": channel_delta}


def layer(x, w, cfg, i):
    spec, eps, pre = cfg["layers"][i], float(cfg["norm"]["eps"]), f"l{i}."
    y = MIXERS[spec["type"]](rms(x, eps) * w[pre + "norm1"].to(F64), w,
                             pre + "mix.", spec["mixer"], eps) \
        * w[pre + "ls1"].to(F64)
    mlp = spec.get("mlp")
    if mlp:
        h2 = rms(x, eps) * w[pre + "norm2"].to(F64)
        f = dense_ff(h2, w, pre + "mlp.") if mlp["kind"] == "dense" \
            else moe_ff(h2, w, pre + "mlp.", mlp)
        y = y + f * w[pre + "ls2"].to(F64)
    return x + y


def layer_order(cfg):
    """[(layer, first of a repeated pass)] in execution order."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(a)]
    for t in range(times):
        order += [(i, t > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(tokens, w, cfg, streams=None):
    """Logits [L, vocab] of one whole sequence. ``streams`` (a list) receives
    the residual stream after every layer run."""
    x0 = embedding(list(tokens), w, cfg)
    x = x0.clone()
    for i, again in layer_order(cfg):
        if again:
            x = x + x0
        x = layer(x, w, cfg, i)
        if streams is not None:
            streams.append(x.clone())
    x = rms(x, float(cfg["norm"]["eps"])) * w["final.norm"].to(F64)
    return lin(w["embed"], x) * float(cfg.get("logit_scale", 1.0))
