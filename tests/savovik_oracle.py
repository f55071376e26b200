"""A plain, slow formulation of the Savovik design's mechanisms, one function
per mechanism, written from its equations for whole sequences (no cache, no
batching, no steps). float64 throughout unless ``dtype`` says otherwise; it
shares no code with the serving path and is what the tests compare against.

Weights arrive as a dict of tensors under their checkpoint names
('l<i>.mix.q', 'l<i>.mlp.up', ...), linear weights stored [out, in].
"""

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def frequencies(rot):
    """Rotation frequency of every pair; 'scaling' with 'original' means the
    three-band rule (long waves slowed by 'factor', short ones kept, a
    blend between), otherwise every frequency is divided by 'factor'."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)],
                     dtype=torch.float64)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor = float(sc["factor"])
    if "original" not in sc:
        return f / factor
    orig, low, high = float(sc["original"]), float(sc["low"]), float(sc["high"])
    out = []
    for fi in f.tolist():
        wave = 2 * math.pi / fi
        if wave < orig / high:
            out.append(fi)
        elif wave > orig / low:
            out.append(fi / factor)
        else:
            s = (orig / wave - low) / (high - low)
            out.append((1 - s) * fi / factor + s * fi)
    return torch.tensor(out, dtype=torch.float64)


def rotate(x, rot, layout, first_pos=0):
    """x [L, heads, dim]; pairs (2i, 2i+1) for 'interleaved', (i, i + dims/2)
    for 'half', among the first rot.dims coordinates."""
    dims = int(rot["dims"])
    L = x.shape[0]
    ang = torch.arange(first_pos, first_pos + L, dtype=torch.float64)[:, None] \
        * frequencies(rot)[None, :]
    c, s = ang.cos()[:, None, :].to(x.dtype), ang.sin()[:, None, :].to(x.dtype)
    out = x.clone()
    if layout == "interleaved":
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    return out


def visible(L, mask_kind, size):
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    see = j <= i
    if mask_kind == "window":
        see = see & (i - j < size)
    elif mask_kind == "chunk":
        see = see & (i // size == j // size)
    return see


def softmax_attention(q, k, v, scale, see, softcap=None):
    """q [L, H, d], k [L, G, d], v [L, G, dv] -> [L, H*dv]."""
    L, H, _ = q.shape
    G = k.shape[1]
    outs = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~see, float("-inf"))
        outs.append(torch.softmax(s, -1) @ v[:, g])
    return torch.cat(outs, -1)


def window_attention_mixer(h, w, pre, m, eps):
    """The 'attention' mixer: no biases, rotate-half rotation with linearly
    scaled frequencies, unit-RMS values, capped scores, sliding window."""
    L = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[pre + "q"].T).reshape(L, H, d)
    k = (h @ w[pre + "k"].T).reshape(L, G, d)
    v = (h @ w[pre + "v"].T).reshape(L, G, dv)
    q, k = rotate(q, m["rot"], "half"), rotate(k, m["rot"], "half")
    v = rms(v, eps)
    o = softmax_attention(q, k, v, float(m["scale"]),
                          visible(L, "window", int(m["mask"]["size"])),
                          float(m["softcap"]))
    return o @ w[pre + "o"].T


def chunk_attention_mixer(h, w, pre, m, eps):
    """The left half of the 'parallel' mixer: biased projections, per-head
    RMS norm of queries and keys, interleaved rotation with three-band
    frequencies, attention inside chunks counted from position 0."""
    L = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(L, H, d)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(L, G, d)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(L, G, dv)
    q = rms(q, eps) * w[pre + "q.norm"]
    k = rms(k, eps) * w[pre + "k.norm"]
    q, k = rotate(q, m["rot"], "interleaved"), rotate(k, m["rot"], "interleaved")
    o = softmax_attention(q, k, v, float(m["scale"]),
                          visible(L, "chunk", int(m["mask"]["size"])))
    return o @ w[pre + "o"].T


def causal_conv(x, w, b):
    """x [L, C]; w [C, taps], last column weighs the current token; zeros
    before the start."""
    L, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + pad[j:j + L] * w[:, j]
    return y + b


def selective_scan_mixer(h, w, pre, m):
    """The right half of the 'parallel' mixer: one state vector per channel."""
    L = h.shape[0]
    inner, N, R = int(m["inner"]), int(m["state"]), int(m["dt_rank"])
    xz = h @ w[pre + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, w[pre + "conv"], w[pre + "conv.b"]))
    p = x @ w[pre + "x"].T
    dt, B, C = p[:, :R], p[:, R:R + N], p[:, R + N:]
    dt = softplus(dt @ w[pre + "dt"].T + w[pre + "dt.b"])
    A = -torch.exp(w[pre + "A_log"])
    S = torch.zeros(inner, N, dtype=h.dtype)
    ys = []
    for t in range(L):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        ys.append(S @ C[t] + w[pre + "D"] * x[t])
    y = torch.stack(ys) * silu(z)
    return y @ w[pre + "o"].T


def parallel_mixer(h, w, pre, m, eps):
    return float(m["left_scale"]) * chunk_attention_mixer(h, w, pre + "left.", m["left"], eps) \
        + float(m["right_scale"]) * selective_scan_mixer(h, w, pre + "right.", m["right"])


def mamba2_mixer(h, w, pre, m, eps):
    """Scalar decay per head, matrix state [N, vdim] per head, gate before a
    grouped RMS norm."""
    L = h.shape[0]
    H, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * P
    p = h @ w[pre + "in"].T
    z = p[:, :inner]
    xbc = silu(causal_conv(p[:, inner:2 * inner + 2 * G * N], w[pre + "conv"],
                           w[pre + "conv.b"]))
    dt = softplus(p[:, 2 * inner + 2 * G * N:] + w[pre + "dt_bias"])
    x = xbc[:, :inner].reshape(L, H, P)
    B = xbc[:, inner:inner + G * N].reshape(L, G, N)
    C = xbc[:, inner + G * N:].reshape(L, G, N)
    a = torch.exp(w[pre + "A_log"])
    ys = torch.zeros(L, H, P, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        for t in range(L):
            S = torch.exp(-a[hd] * dt[t, hd]) * S \
                + dt[t, hd] * B[t, g][:, None] * x[t, hd][None, :]
            ys[t, hd] = S.T @ C[t, g] + w[pre + "D"][hd] * x[t, hd]
    y = ys.reshape(L, inner) * silu(z)
    parts = int(m["norm_groups"])
    y = rms(y.reshape(L, parts, inner // parts), eps).reshape(L, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T


def dense_ff(h, w, pre):
    return gelu_erf(h @ w[pre + "up"].T) @ w[pre + "down"].T


def mixer(kind, h, w, pre, m, eps):
    if kind == "attention":
        return window_attention_mixer(h, w, pre, m, eps)
    if kind == "parallel":
        return parallel_mixer(h, w, pre, m, eps)
    if kind == "mamba2":
        return mamba2_mixer(h, w, pre, m, eps)
    raise ValueError(kind)


def layer(x, w, cfg, i):
    """One layer: a shared norm, mixer and feed-forward side by side, each
    scaled by a sigmoid gate computed from the normed input."""
    spec = cfg["layers"][i]
    src = spec.get("weights_of", i)
    pre = f"l{src}."
    eps = float(cfg["norm"]["eps"])
    h = norm_one_plus(x, w[pre + "norm1"], eps)
    g1 = torch.sigmoid(h @ w[pre + "rg1"].T + w[pre + "rg1.b"])
    out = g1 * mixer(spec["type"], h, w, pre + "mix.", spec["mixer"], eps)
    if spec.get("mlp"):
        g2 = torch.sigmoid(h @ w[pre + "rg2"].T + w[pre + "rg2.b"])
        out = out + g2 * dense_ff(h, w, pre + "mlp.")
    return x + out


def forward(tokens, w, cfg, dtype=torch.float64, streams=None):
    """Logits [L, vocab] of one whole sequence; ``streams`` (a list) receives
    the residual stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i in range(len(cfg["layers"])):
        x = layer(x, w, cfg, i)
        if streams is not None:
            streams.append(x.clone())
    x = norm_one_plus(x, w["final.norm"], float(cfg["norm"]["eps"]))
    return x @ w["head"].T
