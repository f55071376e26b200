"""Linear recurrences with a matrix state per head, for ragged batches.

A head carries ``S`` ([dim, vdim], fp32, one per request slot). Per token, in
this order:

    S <- decay * S                  decay: one number per head, or one per key
                                    channel (it then scales the rows of S)
    u  = v                          plain form ("gla")
    u  = beta * (v - S^T k)         delta-rule form (beta given)
    S <- S + k u^T
    o  = S^T q                      (sees this token's write)

so a step that brings only a portion of a sequence continues from the slot's
state exactly where the previous step stopped, and a result cannot depend on
where a sequence was cut. Everything is fp32; q/k/v may arrive in the compute
dtype (they are projections) and are widened on load.

Around the scan:

* ``delta_prep``: the gated delta rule's inputs from its fused projection
  (short convolution + SiLU on q, k, v with carried tails; q and k scaled to
  unit length per head; ``beta = sigmoid(b)``;
  ``decay = exp(-exp(A_log) * softplus(a + dt_bias))``).
* ``ssd_prep``: the scalar-decay state-space form's inputs from its fused
  projection ``z | x | B | C | dt`` (short convolution with bias + SiLU on
  x|B|C with carried tails; ``dt = softplus(dt + dt_bias)``;
  ``decay = exp(-exp(A_log) * dt)``; the scan's ``v`` is ``dt * x``, its keys
  are B and its queries C, shared by the heads of a group).
* ``gate_group_norm``: the read-out plus the skip ``D * x``, times
  ``silu(gate)``, then an RMS norm over equal parts of the row, times a weight.
* ``sigmoid_pow``: ``sigmoid(z + bias) ** (1 / tau)`` for per-channel decays.
* ``softplus_decay``: ``exp(-exp(A_log_h) * softplus(z + bias))`` per head and
  key channel (the delta rule with a decay of its own for every row of S).
* ``head_norm_gate``: per-head RMS norm of the read-out times a weight shared
  by the heads, times ``silu(gate)`` or ``sigmoid(gate)``.
"""

import torch
import torch.nn.functional as F

from .causal_conv import conv_silu_ragged

UNIT_EPS = 1e-6


def _sk():
    from . import serving_kernels
    return serving_kernels


def unit_heads(x, scale=1.0):
    """x [T, n, d] fp32 -> x / sqrt(sum(x^2) + 1e-6) * scale per head."""
    return x * torch.rsqrt(x.pow(2).sum(-1, keepdim=True) + UNIT_EPS) * scale


def delta_prep(proj, batch, conv_w, conv_state, a_log, dt_bias, kv_heads,
               heads, dim, vdim, beta_col=None, a_col=None):
    """proj [T, ...] starts with q | k | v; by default the row goes on
    ``| gate | b | a`` (the gate columns are left for ``head_norm_gate``).
    ``beta_col`` / ``a_col`` name the first of the ``heads`` columns of b and
    of a in other layouts; ``a_col=-1`` makes no per-head decay here (the
    caller has one per key channel, see ``softplus_decay``) and returns None
    for it. conv_w [2*kv_heads*dim + heads*vdim, taps] and
    conv_state [slots, taps-1, same] cover the q|k|v columns.
    Returns fp32 q [T, kv_heads, dim] (unit length times dim^-1/2),
    k [T, kv_heads, dim] (unit length), v [T, heads, vdim], beta [T, heads],
    decay [T, heads]."""
    T = proj.shape[0]
    nqk, nv = kv_heads * dim, heads * vdim
    C = 2 * nqk + nv
    if beta_col is None:
        assert proj.shape[1] == C + nv + 2 * heads
        beta_col = C + nv
    if a_col is None:
        a_col = beta_col + heads
    assert conv_w.shape[0] == C
    if proj.is_cuda and _sk().enabled():
        return _sk().delta_prep(proj, batch, conv_w, conv_state, a_log,
                                dt_bias, kv_heads, heads, dim, vdim,
                                beta_col, a_col)
    y = conv_silu_ragged(proj[:, :C], conv_w, conv_state, batch)
    q = unit_heads(y[:, :nqk].reshape(T, kv_heads, dim), dim ** -0.5)
    k = unit_heads(y[:, nqk:2 * nqk].reshape(T, kv_heads, dim))
    v = y[:, 2 * nqk:].reshape(T, heads, vdim)
    beta = torch.sigmoid(proj[:, beta_col:beta_col + heads].float())
    decay = None
    if a_col >= 0:
        dt = F.softplus(proj[:, a_col:a_col + heads].float()
                        + dt_bias.float())
        decay = torch.exp(-torch.exp(a_log.float()) * dt)
    return q.contiguous(), k.contiguous(), v.contiguous(), beta, decay


def softplus_decay(z, bias, a_log, heads):
    """Per head and key channel: ``exp(-exp(a_log_h) * softplus(z + bias))``
    in fp32. z [T, heads*dim] (a projection, may be a column slice),
    bias [heads*dim], a_log [heads]. Returns [T, heads, dim]."""
    if z.is_cuda and _sk().enabled():
        return _sk().softplus_decay(z, bias, a_log, heads)
    T, C = z.shape
    dt = F.softplus(z.float() + bias.float()).view(T, heads, C // heads)
    return torch.exp(-torch.exp(a_log.float())[None, :, None] * dt)


def sigmoid_pow(z, bias, inv_tau):
    """``sigmoid(z + bias) ** inv_tau`` in fp32, evaluated as
    ``exp(inv_tau * log_sigmoid(.))``."""
    if z.is_cuda and _sk().enabled():
        return _sk().sigmoid_pow(z, bias, inv_tau)
    return torch.exp(inv_tau * F.logsigmoid(z.float() + bias.float()))


def linear_scan(q, k, v, decay, beta, state, batch, q_scale=1.0):
    """q, k [T, G, dim]; v [T, H, vdim] (head h reads q/k head h // (H/G));
    decay [T, H] or [T, H, dim] fp32; beta [T, H] fp32 or None;
    state [slots, H, dim, vdim] fp32, updated in place. q, k, v may be
    strided views (last axis contiguous). Returns o [T, H, vdim] fp32."""
    T, G, dim = q.shape
    H, vdim = v.shape[1], v.shape[2]
    assert H % G == 0 and state.dtype == torch.float32
    assert state.shape[1:] == (H, dim, vdim)
    assert decay.shape in ((T, H), (T, H, dim))
    if q.is_cuda and _sk().enabled():
        return _sk().linear_scan(q, k, v, decay, beta, state, batch, q_scale)
    rep = H // G
    qf = (q.float() * q_scale).repeat_interleave(rep, 1)
    kf = k.float().repeat_interleave(rep, 1)
    vf = v.float()
    dec = decay.float()
    dec = dec[:, :, None, None] if dec.dim() == 2 else dec[:, :, :, None]
    out = torch.empty(T, H, vdim, dtype=torch.float32, device=q.device)
    at = 0
    for slot, count in zip(batch.slots, batch.counts):
        S = state[slot]
        for t in range(at, at + count):
            S = dec[t] * S
            u = vf[t]
            if beta is not None:
                u = beta[t, :, None] * (u - torch.einsum("hdv,hd->hv", S,
                                                         kf[t]))
            S = S + kf[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S
        at += count
    return out


def head_norm_gate(o, weight, gate, eps, out_dtype, act="silu"):
    """o [T, H, vdim] fp32; weight [vdim]; gate [T, H*vdim] pre-activation
    (may be a column slice). Returns
    ``o / sqrt(mean_v(o^2) + eps) * weight * act(gate)`` as
    [T, H*vdim] ``out_dtype``; ``act`` is "silu" or "sigmoid"."""
    T, H, vdim = o.shape
    if act not in ("silu", "sigmoid"):
        raise ValueError(f"unknown gate activation {act!r}")
    if o.is_cuda and _sk().enabled():
        return _sk().head_norm_gate(o, weight, gate, eps, out_dtype, act)
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    g = F.silu(gate.float()) if act == "silu" else torch.sigmoid(gate.float())
    return (y.reshape(T, H * vdim) * g).to(out_dtype)


def ssd_prep(proj, batch, conv_w, conv_b, conv_state, a_log, dt_bias, heads,
             groups, state, vdim):
    """proj [T, 2*heads*vdim + 2*groups*state + heads] =
    z | x | B | C | dt (the z columns are left for ``gate_group_norm``).
    conv_w [heads*vdim + 2*groups*state, taps], conv_b and conv_state
    [slots, taps-1, same] cover the x|B|C columns.
    Returns fp32 C [T, groups, state], B [T, groups, state],
    v = dt * x [T, heads, vdim], x [T, heads, vdim], decay [T, heads]."""
    T = proj.shape[0]
    inner, gn = heads * vdim, groups * state
    C = inner + 2 * gn
    assert proj.shape[1] == 2 * inner + 2 * gn + heads and conv_w.shape[0] == C
    if proj.is_cuda and _sk().enabled():
        return _sk().ssd_prep(proj, batch, conv_w, conv_b, conv_state, a_log,
                              dt_bias, heads, groups, state, vdim)
    y = conv_silu_ragged(proj[:, inner:inner + C], conv_w, conv_state, batch,
                         conv_b)
    x = y[:, :inner].reshape(T, heads, vdim)
    Bk = y[:, inner:inner + gn].reshape(T, groups, state)
    Cq = y[:, inner + gn:].reshape(T, groups, state)
    dt = F.softplus(proj[:, inner + C:].float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * dt)
    v = dt[:, :, None] * x
    return Cq.contiguous(), Bk.contiguous(), v, x.contiguous(), decay


def gate_group_norm(o, x, skip, gate, weight, parts, eps, out_dtype):
    """o, x [T, H, vdim] fp32; skip [H]; gate [T, H*vdim] pre-activation (may
    be a column slice); weight [H*vdim]. With ``y = (o + skip_h * x) *
    silu(gate)``, returns ``y / sqrt(mean_part(y^2) + eps) * weight`` where
    the mean runs over each of ``parts`` equal pieces of the row, as
    [T, H*vdim] ``out_dtype``."""
    T, H, vdim = o.shape
    n = H * vdim
    assert n % parts == 0 and weight.numel() == n
    if o.is_cuda and _sk().enabled():
        return _sk().gate_group_norm(o, x, skip, gate, weight, parts, eps,
                                     out_dtype)
    y = (o + skip.float()[None, :, None] * x).reshape(T, n) \
        * F.silu(gate.float())
    y = y.reshape(T, parts, n // parts)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, n) * weight.float()).to(out_dtype)
