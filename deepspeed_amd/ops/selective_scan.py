"""Selective scan: a diagonal state-space recurrence with one state VECTOR
per channel and input-dependent step sizes, for ragged batches.

Channel c of a sequence carries ``S[c, :]`` ([state], fp32, per request slot).
Per token, with ``dt_c = softplus(dt_pre_c + dt_bias_c)`` and
``A = -exp(A_log)`` ([channels, state]):

    S[c, n] <- exp(dt_c * A[c, n]) * S[c, n] + dt_c * x_c * B_n
    y_c      = sum_n S[c, n] * C_n + D_c * x_c
    out_c    = y_c * silu(z_c) * out_scale

B and C ([state] per token) are shared by all channels. Step sizes, decays,
the state and the sums are fp32; x, B, C and z may arrive in the compute dtype
(projections and a convolution's output) and are widened on load. A step that
brings a portion of a sequence continues from the slot's state, and the sum
over ``n`` runs in a fixed order, so a result does not depend on where a
sequence was cut.
"""

import torch
import torch.nn.functional as F


def _sk():
    from . import serving_kernels
    return serving_kernels


def selective_scan(x, dt_pre, dt_bias, a_log, B, C, skip, z, state, batch,
                   out_dtype=None, out_scale=1.0, out=None):
    """x [T, channels]; dt_pre [T, channels] fp32; dt_bias, skip [channels];
    a_log [channels, n]; B, C [T, n]; z [T, channels]; state
    [slots, channels, n] fp32, updated in place. x, B, C, z may be column
    slices (rows contiguous). Returns [T, channels] ``out_dtype`` (x's by
    default), written into ``out`` when given (a view with contiguous rows)."""
    T, ch = x.shape
    n = a_log.shape[1]
    out_dtype = out_dtype or x.dtype
    assert state.dtype == torch.float32 and state.shape[1:] == (ch, n)
    assert B.shape == (T, n) and C.shape == (T, n) and z.shape == (T, ch)
    assert dt_pre.shape == (T, ch) and dt_pre.dtype == torch.float32
    if out is None:
        out = torch.empty(T, ch, dtype=out_dtype, device=x.device)
    assert out.shape == (T, ch) and out.stride(1) == 1 \
        and out.dtype == out_dtype
    if x.is_cuda and _sk().enabled():
        return _sk().selective_scan(x, dt_pre, dt_bias, a_log, B, C, skip, z,
                                    state, batch, out_scale, out)
    A = -torch.exp(a_log.float())
    dt = F.softplus(dt_pre + dt_bias.float())
    xf, Bf, Cf = x.float(), B.float(), C.float()
    gate = F.silu(z.float())
    at = 0
    for slot, count in zip(batch.slots, batch.counts):
        S = state[slot]
        for t in range(at, at + count):
            S = torch.exp(dt[t][:, None] * A) * S \
                + (dt[t] * xf[t])[:, None] * Bf[t][None, :]
            y = S @ Cf[t] + skip.float() * xf[t]
            out[t] = (y * gate[t] * out_scale).to(out_dtype)
        state[slot] = S
        at += count
    return out
