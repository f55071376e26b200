"""Multi-head attention over paged K/V rows with a sliding window that also
keeps a sequence's first tokens, for ragged batches.

Every token caches ONE row per stream: ``[k (G x dim) ; v (G x vdim)]`` for the
G key/value heads; query head h reads key/value head ``h // (H / G)``. Position
i of a sequence sees position j when ``j <= i`` and (``i - j < window`` or
``j < keep_first``); kept tokens stay where they are (their rows were rotated
at their true positions). ``window <= 0`` means no window (plain causal).
Scores, softmax and the weighted sum are fp32.

Two more masks and a score transform share the kernels: ``chunk > 0`` lets
position i see j only when ``i // chunk == j // chunk`` (chunks counted from a
sequence's position 0, wherever a prompt was cut); ``softcap > 0`` replaces a
scaled score s by ``softcap * tanh(s / softcap)`` before the softmax.

``attn_prep`` finishes a step's fused q|k|v projection: an RMS norm of queries
and keys (``norm="whole"``: over the WHOLE query projection, all heads at
once, one weight per coordinate, and over the whole key projection;
``norm="head"``: per head over ``dim`` with one weight of size ``dim`` shared
by the heads; ``None``: no norm), rotation of the first ``rot_dims``
coordinates of every head (``layout="interleaved"`` pairs 2i with 2i+1,
``"half"`` pairs i with i + rot_dims/2), optionally each value head divided by
its root mean square (``v_unit_eps``), and the write of the new rows into the
pool. A layer that borrows another layer's rows passes ``own_kv=False``: its
projection holds queries only and nothing is written.
"""

import torch

from .rope import rope_half_, rope_interleaved_


def _sk():
    from . import serving_kernels
    return serving_kernels


def _rms_all(x, w, eps):
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()


def _qk_norm(x, w, eps, norm, n_heads, dim):
    T = x.shape[0]
    if norm == "whole":
        return _rms_all(x, w, eps).reshape(T, n_heads, dim)
    xf = x.float().reshape(T, n_heads, dim)
    if norm == "head":
        return _rms_all(xf, w, eps)
    return xf.clone()           # rotated in place: never the caller's rows


def attn_prep(proj, batch, pool, q_norm_w, k_norm_w, eps, heads, kv_heads,
              dim, vdim, rot_dims, cos, sin, own_kv=True, norm="whole",
              layout="interleaved", v_unit_eps=None):
    """proj [T, heads*dim (+ kv_heads*dim + kv_heads*vdim)] = q | k | v (may
    be a column slice of a wider projection). Returns q [T, heads, dim] in
    proj's dtype; with ``own_kv`` the rows [k ; v] of this step's tokens are
    written into ``pool`` ([blocks, block_size, kv_heads*(dim+vdim)])."""
    T = proj.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    assert proj.shape[1] == nq + (nk + nv if own_kv else 0)
    assert norm in ("whole", "head", None) and layout in ("interleaved", "half")
    if proj.is_cuda and _sk().enabled():
        return _sk().attn_prep(proj, batch, pool, q_norm_w, k_norm_w, eps,
                               heads, kv_heads, dim, vdim, rot_dims, cos, sin,
                               own_kv, norm, layout, v_unit_eps)
    rotate = rope_interleaved_ if layout == "interleaved" else rope_half_
    q = _qk_norm(proj[:, :nq], q_norm_w, eps, norm, heads, dim)
    if rot_dims:
        rotate(q, batch.tok_pos, cos, sin, rot_dims)
    if own_kv:
        k = _qk_norm(proj[:, nq:nq + nk], k_norm_w, eps, norm, kv_heads, dim)
        if rot_dims:
            rotate(k, batch.tok_pos, cos, sin, rot_dims)
        v = proj[:, nq + nk:]
        if v_unit_eps is not None:
            vf = v.float().reshape(T, kv_heads, vdim)
            v = (vf * torch.rsqrt(vf.pow(2).mean(-1, keepdim=True)
                                  + v_unit_eps)).reshape(T, nv)
        rows = torch.cat([k.reshape(T, nk).to(pool.dtype),
                          v.to(pool.dtype)], -1)
        pool.view(-1, nk + nv)[batch.tok_row.long()] = rows
    return q.to(proj.dtype)


def window_mask(qpos, kpos, window, keep_first, chunk=0):
    """[len(qpos), len(kpos)] bool: which keys each query sees."""
    d = qpos[:, None] - kpos[None, :]
    near = d >= 0
    if window > 0:
        near = near & ((d < window) | (kpos[None, :] < keep_first))
    if chunk > 0:
        near = near & ((qpos[:, None] // chunk == kpos[None, :] // chunk)
                       | (kpos[None, :] < keep_first))
    return near


def window_attention(q, pool, batch, kv_heads, dim, vdim, scale, window=0,
                     keep_first=0, path=None, chunk=0, softcap=0.0,
                     out_scale=1.0, out=None):
    """q [T, heads, dim]; pool holds every sequence's rows INCLUDING this
    step's. Returns [T, heads*vdim] in q's dtype, times ``out_scale``;
    ``out`` (a [T, heads*vdim] view whose rows are contiguous, e.g. a column
    slice of a wider buffer) receives the result when given."""
    T, H, _ = q.shape
    assert H % kv_heads == 0 and pool.shape[-1] == kv_heads * (dim + vdim)
    assert not (window > 0 and chunk > 0), "one mask per layer"
    if out is None:
        out = torch.empty(T, H * vdim, dtype=q.dtype, device=q.device)
    assert out.shape == (T, H * vdim) and out.stride(1) == 1
    if q.is_cuda and _sk().enabled():
        return _sk().window_attention(q, pool, batch, kv_heads, dim, vdim,
                                      scale, window, keep_first, path, chunk,
                                      softcap, out_scale, out)
    bs = batch.block_size
    rows = pool.view(-1, pool.shape[-1])
    rep = H // kv_heads
    at = 0
    for i, (st, cnt) in enumerate(zip(batch.starts, batch.counts)):
        L = st + cnt
        pos = torch.arange(L, device=q.device)
        ctx = rows[batch.block_table[i].long()[pos // bs] * bs + pos % bs]
        ctx = ctx.float()
        k = ctx[:, :kv_heads * dim].reshape(L, kv_heads, dim) \
            .repeat_interleave(rep, 1)
        v = ctx[:, kv_heads * dim:].reshape(L, kv_heads, vdim) \
            .repeat_interleave(rep, 1)
        s = torch.einsum("thd,lhd->htl", q[at:at + cnt].float(), k) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        see = window_mask(st + torch.arange(cnt, device=q.device), pos,
                          window, keep_first, chunk)
        s = s.masked_fill(~see[None], float("-inf"))
        p = torch.softmax(s, -1)
        o = torch.einsum("htl,lhv->thv", p, v) * out_scale
        out[at:at + cnt] = o.reshape(cnt, H * vdim).to(q.dtype)
        at += cnt
    return out
