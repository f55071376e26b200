"""Feed-forward activations used by the serving models (beside swiglu/geglu).

* ``xielu(z, p, q)``: for z > 0 ``softplus(p) z^2 + z/2``; otherwise
  ``(1/2 + softplus(q)) (exp(z) - 1 - z) + z/2``. p and q are learned
  numbers of the layer.
* ``clamped_swiglu(gu, limit)``: with ``g = min(gate, limit)`` and
  ``u = clamp(up, -limit, limit)``: ``g * sigmoid(1.702 g) * (u + 1)``;
  ``gu`` holds gate and up side by side ([T, 2F] -> [T, F]).
* ``glu(gu, act)``: ``act(gate) * up`` with ``act`` "silu" or "gelu_tanh"
  (``0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))``), same layout.
* ``act_rows(z, act)``: a plain activation of a projection, ``act`` one of
  "gelu_erf" (``0.5 z (1 + erf(z / sqrt 2))``), "gelu_tanh", "silu"; ``z`` may
  be a column slice of a wider projection.
All evaluate in fp32 and round once.
"""

import torch
import torch.nn.functional as F

def _sk():
    from . import serving_kernels
    return serving_kernels


SWISH_SLOPE = 1.702


def xielu(z, pq):
    """z [T, F]; pq a 2-element fp32 tensor (p, q)."""
    if z.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.xielu(z, pq)
    zf = z.float()
    a = F.softplus(pq[0].float())
    b = 0.5 + F.softplus(pq[1].float())
    neg = b * (torch.expm1(zf.clamp(max=0)) - zf) + 0.5 * zf
    pos = a * zf * zf + 0.5 * zf
    return torch.where(zf > 0, pos, neg).to(z.dtype)


def clamped_swiglu(gu, limit):
    if gu.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.clamped_swiglu(gu, limit)
    f = gu.shape[-1] // 2
    g = gu[..., :f].float().clamp(max=limit)
    u = gu[..., f:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(SWISH_SLOPE * g) * (u + 1)).to(gu.dtype)


GLU_ACTS = ("silu", "gelu_tanh")


def glu(gu, act):
    """gu [..., 2F] = gate | up -> act(gate) * up as [..., F]."""
    if act not in GLU_ACTS:
        raise ValueError(f"unknown gate activation {act!r}")
    if gu.is_cuda and _sk().enabled():
        return _sk().glu(gu, GLU_ACTS.index(act))
    f = gu.shape[-1] // 2
    g, u = gu[..., :f].float(), gu[..., f:].float()
    a = F.silu(g) if act == "silu" else F.gelu(g, approximate="tanh")
    return (a * u).to(gu.dtype)


ROW_ACTS = ("gelu_erf", "gelu_tanh", "silu")


def act_rows(z, act):
    """z [T, F] (rows contiguous, any row stride) -> act(z), contiguous."""
    if act not in ROW_ACTS:
        raise ValueError(f"unknown activation {act!r}")
    if z.is_cuda and _sk().enabled():
        return _sk().act_rows(z, ROW_ACTS.index(act))
    zf = z.float()
    if act == "gelu_erf":
        y = F.gelu(zf)
    elif act == "gelu_tanh":
        y = F.gelu(zf, approximate="tanh")
    else:
        y = F.silu(zf)
    return y.to(z.dtype)
