"""Short depthwise causal convolution over time with carried state, for
ragged serving batches.

``y_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j)`` per channel, with zeros
before a sequence's start. A sequence's last ``taps - 1`` inputs are its
carried state (``state[slot]``, oldest first), so a step that brings only a
portion of a sequence continues exactly where the previous one stopped.

The serving form fuses the preceding single-gain RMS norm: the kernel reads
the fp32 residual stream, normalises in fp32, rounds the normed input ``h``
to the compute dtype (that rounded value is also what the state keeps, so
the result does not depend on where a sequence was cut), and convolves.
"""

import torch


def _sk():
    from . import serving_kernels
    return serving_kernels


def _norm(x, gain, eps, dtype):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
            * gain.float().reshape(())).to(dtype)


def norm_conv_ragged(x, gain, eps, conv_w, state, batch, out_dtype,
                     sumsq=None):
    """x [T, C] fp32 residual; conv_w [C, taps]; state [slots, taps-1, C]
    (updated in place); batch: RaggedBatch. Returns h + conv(h) as
    [T, C] ``out_dtype``. ``sumsq`` ([T] fp32, from ``residual_add_stats``)
    spares the kernel its own reduction over x."""
    if x.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.norm_conv_ragged(x, gain, eps, conv_w, state, batch,
                                   out_dtype, sumsq)
    taps = conv_w.shape[1]
    h = _norm(x, gain, eps, out_dtype)
    out = torch.empty_like(h)
    wf = conv_w.float()
    at = 0
    for slot, count in zip(batch.slots, batch.counts):
        hist = torch.cat([state[slot], h[at:at + count]], 0).float()
        win = hist.unfold(0, taps, 1)                 # [count, C, taps]
        out[at:at + count] = (hist[taps - 1:] +
                              (win * wf).sum(-1)).to(out_dtype)
        if taps > 1:
            state[slot] = hist[-(taps - 1):].to(state.dtype)
        at += count
    return out


def residual_add_stats(x, delta):
    """x += delta (fp32 stream, delta in the compute dtype), in place. On the
    GPU the same pass returns every row's sum of squares for the norm that
    follows; the eager path returns None and the norm reduces by itself."""
    if x.is_cuda and _sk().enabled():
        return _sk().residual_add_stats(x, delta)
    x.add_(delta)
    return None


def conv_silu_ragged(x, conv_w, state, batch, bias=None, out_dtype=None):
    """Short causal convolution per channel followed by SiLU:
    ``silu(sum_j w[:, j] * x_(t - taps + 1 + j) (+ bias))`` with zeros before
    a sequence's start (the last column weighs the current token).
    x [T, C] (may be a column slice of a wider projection), conv_w [C, taps],
    state [slots, taps-1, C] in x's dtype: a sequence's last ``taps - 1``
    inputs, oldest first, updated in place. Sums and SiLU are fp32; returns
    [T, C] fp32, or rounded once to ``out_dtype``."""
    out_dtype = out_dtype or torch.float32
    if x.is_cuda and _sk().enabled():
        return _sk().conv_silu_ragged(x, conv_w, state, batch, bias,
                                      out_dtype)
    taps = conv_w.shape[1]
    wf = conv_w.float()
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    at = 0
    for slot, count in zip(batch.slots, batch.counts):
        hist = torch.cat([state[slot].to(x.dtype), x[at:at + count]], 0)
        win = hist.float().unfold(0, taps, 1)          # [count, C, taps]
        acc = (win * wf).sum(-1)
        if bias is not None:
            acc = acc + bias.float()
        out[at:at + count] = torch.nn.functional.silu(acc).to(out_dtype)
        if taps > 1:
            state[slot] = hist[-(taps - 1):].to(state.dtype)
        at += count
    return out
