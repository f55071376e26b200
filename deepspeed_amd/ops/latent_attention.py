"""Latent (compressed-KV) attention over a paged cache, for ragged batches.

Every token caches ONE row shared by all heads: ``[c ; k_rot]`` with ``c`` the
normed latent (``rank`` numbers) and ``k_rot`` the rotated key part
(``rot`` numbers). Per head the unrotated key is ``W_uk c`` and the value
``W_uv c``; both up-projections are folded into the query and the output
instead of being applied to the cache:

    score(i, j) = ((W_uk^T q_nope_i) . c_j + q_rot_i . k_rot_j) * scale
    out_i       = W_uv (sum_j p_ij c_j)

so the attention kernel is multi-query attention whose key is the cached row
and whose value is its first ``rank`` entries. Scores, softmax and the
weighted sum are fp32. Position i of a sequence sees rows 0..i, or with a
``window`` only rows i-window+1..i. A ``sink`` (one fp32 logit per head) joins
the softmax's denominator as ``exp(sink_h)``: it has no key and no value and
is not scaled, so the weights of a row sum to less than one.

``latent_prep`` finishes the input projections of a step: norm of the latent,
rotation of the shared key part and of the queries' rotated parts (pairs of
neighbours, or coordinate i with i + rot_dims/2), the output gate's sigmoid,
and the write of the new rows into the pool. ``rot`` may be 0 (no rotated
part: the row is the latent alone) and the gate may be absent.
"""

import torch

from .rope import rope_half_, rope_interleaved_


def _sk():
    from . import serving_kernels
    return serving_kernels


def latent_prep(proj, batch, pool, norm_w, eps, heads, dim, rot, rank,
                rot_dims, cos, sin, layout="interleaved"):
    """proj [T, heads*(dim+rot) + rank + rot + heads] = q | latent | k_rot |
    gate logits. See ``latent_prep_parts``."""
    nq = heads * (dim + rot)
    return latent_prep_parts(proj[:, :nq], proj[:, nq:nq + rank + rot],
                             proj[:, nq + rank + rot:], batch, pool, norm_w,
                             eps, heads, dim, rot, rank, rot_dims, cos, sin,
                             layout)


def latent_prep_parts(q, kv, gate_z, batch, pool, norm_w, eps, heads, dim,
                      rot, rank, rot_dims, cos, sin, layout="interleaved"):
    """q [T, heads*(dim+rot)] (per head: unrotated, then rotated part),
    kv [T, rank+rot] = latent | k_rot, gate_z [T, heads] logits or None; each
    may be a column slice of a wider projection. Writes the new rows
    ``[norm(latent) ; rotated k_rot]`` into ``pool`` ([blocks, bs, rank+rot]).
    Returns q_nope [heads, T, dim] (contiguous), q_rot [T, heads, rot] (None
    when rot is 0), gate = sigmoid(gate_z) [T, heads] fp32 (None without)."""
    if q.is_cuda and _sk().enabled():
        return _sk().latent_prep(q, kv, gate_z, batch, pool, norm_w, eps,
                                 heads, dim, rot, rank, rot_dims, cos, sin,
                                 layout)
    T = q.shape[0]
    turn = {"interleaved": rope_interleaved_, "half": rope_half_}[layout]
    q = q.reshape(T, heads, dim + rot)
    lat = kv[:, :rank].float()
    c = lat * torch.rsqrt(lat.pow(2).mean(-1, keepdim=True) + eps) \
        * norm_w.float()
    rows, q_rot = [c.to(pool.dtype)], None
    if rot:
        kr = kv[:, rank:].clone()
        q_rot = q[..., dim:].clone()
        if rot_dims:
            turn(kr, batch.tok_pos, cos, sin, rot_dims)
            turn(q_rot, batch.tok_pos, cos, sin, rot_dims)
        rows.append(kr.to(pool.dtype))
    pool.view(-1, rank + rot)[batch.tok_row.long()] = torch.cat(rows, -1)
    gate = None if gate_z is None else torch.sigmoid(gate_z.float())
    q_nope = q[..., :dim].transpose(0, 1).contiguous()
    return q_nope, q_rot, gate


def latent_attention(q_lat, q_rot, pool, batch, rank, scale, window=0,
                     sink=None):
    """q_lat [heads, T, rank], q_rot [T, heads, rot] or None; pool holds every
    sequence's rows INCLUDING this step's. ``window`` > 0: a query at position
    i sees positions j with 0 <= i - j < window. ``sink`` [heads] fp32 or None.
    Returns [heads, T, rank]."""
    if q_lat.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.latent_attention(q_lat, q_rot, pool, batch, rank, scale,
                                   window=window, sink=sink)
    bs = batch.block_size
    rows = pool.view(-1, pool.shape[-1])
    out = torch.empty_like(q_lat)
    at = 0
    for i, (st, cnt) in enumerate(zip(batch.starts, batch.counts)):
        L = st + cnt
        pos = torch.arange(L, device=q_lat.device)
        ctx = rows[batch.block_table[i].long()[pos // bs] * bs + pos % bs]
        ctx = ctx.float()
        s = torch.einsum("htr,lr->htl", q_lat[:, at:at + cnt].float(),
                         ctx[:, :rank])
        if q_rot is not None:
            s = s + torch.einsum("thd,ld->htl", q_rot[at:at + cnt].float(),
                                 ctx[:, rank:])
        s = s * scale
        qpos = st + torch.arange(cnt, device=q_lat.device)
        hidden = pos[None, None, :] > qpos[None, :, None]
        if window > 0:
            hidden = hidden | (pos[None, None, :] <= qpos[None, :, None]
                               - window)
        s = s.masked_fill(hidden, float("-inf"))
        if sink is not None:
            sk_ = sink.float().view(-1, 1, 1).expand(-1, cnt, 1)
            p = torch.softmax(torch.cat([s, sk_], -1), -1)[..., :-1]
        else:
            p = torch.softmax(s, -1)
        out[:, at:at + cnt] = torch.einsum("htl,lr->htr", p,
                                           ctx[:, :rank]).to(out.dtype)
        at += cnt
    return out


def gate_merge_heads(o, gate=None):
    """o [heads, T, v], gate [T, heads] fp32 or None -> [T, heads*v] (o's
    dtype): heads side by side per token, each scaled by its gate."""
    if o.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.gate_merge_heads(o, gate)
    H, T, v = o.shape
    y = o.float().transpose(0, 1)
    if gate is not None:
        y = y * gate[:, :, None]
    return y.to(o.dtype).reshape(T, H * v)
