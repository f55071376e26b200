"""RMSNorm / LayerNorm modules backed by the CDNA4 HIP kernels.

Kernel parity targets: reference rms_norm.cu / layer_norm.cu (inference) and
normalize_kernels.cu (training fwd+bwd). CPU falls back to a numerically
matching torch implementation (fp32 math internally, like the kernels).
"""

import torch

from ._loader import get_ext


class _RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        ext = get_ext()
        x = x.contiguous()
        if ext is not None and x.is_cuda:
            y, invrms, _ = ext.norm_fwd(x, weight.contiguous(), None, eps, False)
        else:
            xf = x.float()
            invrms = torch.rsqrt(xf.pow(2).mean(-1) + eps)
            y = (xf * invrms.unsqueeze(-1) * weight.float()).to(x.dtype)
            invrms = invrms.reshape(-1)
        ctx.save_for_backward(x, weight, invrms)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, invrms = ctx.saved_tensors
        ext = get_ext()
        dy = dy.contiguous()
        if ext is not None and x.is_cuda:
            dx, dw, _ = ext.norm_bwd(dy, x, weight.contiguous(), invrms, None,
                                     False)
        else:
            H = x.shape[-1]
            xf = x.float().reshape(-1, H)
            dyf = dy.float().reshape(-1, H)
            inv = invrms.unsqueeze(-1)
            xhat = xf * inv
            dyw = dyf * weight.float()
            dot = (dyw * xhat).mean(-1, keepdim=True)
            dx = ((dyw - xhat * dot) * inv).reshape(x.shape).to(x.dtype)
            dw = (dyf * xhat).sum(0)
        return dx, dw.to(weight.dtype), None


class _LayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        ext = get_ext()
        x = x.contiguous()
        if ext is not None and x.is_cuda:
            y, invrms, mean = ext.norm_fwd(
                x, weight.contiguous(),
                bias.contiguous() if bias is not None else None, eps, True)
        else:
            xf = x.float()
            mean = xf.mean(-1)
            var = xf.var(-1, unbiased=False)
            invrms = torch.rsqrt(var + eps)
            y = ((xf - mean.unsqueeze(-1)) * invrms.unsqueeze(-1) *
                 weight.float())
            if bias is not None:
                y = y + bias.float()
            y = y.to(x.dtype)
            invrms, mean = invrms.reshape(-1), mean.reshape(-1)
        ctx.save_for_backward(x, weight, invrms, mean)
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, invrms, mean = ctx.saved_tensors
        ext = get_ext()
        dy = dy.contiguous()
        if ext is not None and x.is_cuda:
            dx, dw, db = ext.norm_bwd(dy, x, weight.contiguous(), invrms, mean,
                                      True)
        else:
            H = x.shape[-1]
            xf = x.float().reshape(-1, H)
            dyf = dy.float().reshape(-1, H)
            inv = invrms.unsqueeze(-1)
            xhat = (xf - mean.unsqueeze(-1)) * inv
            dyw = dyf * weight.float()
            dot = (dyw * xhat).mean(-1, keepdim=True)
            dsum = dyw.mean(-1, keepdim=True)
            dx = ((dyw - dsum - xhat * dot) * inv).reshape(x.shape).to(x.dtype)
            dw = (dyf * xhat).sum(0)
            db = dyf.sum(0)
        grad_bias = db.to(weight.dtype) if ctx.has_bias else None
        return dx, dw.to(weight.dtype), grad_bias, None


def rms_norm(x, weight, eps=1e-6):
    return _RMSNormFn.apply(x, weight, eps)


def layer_norm(x, weight, bias=None, eps=1e-5):
    return _LayerNormFn.apply(x, weight, bias, eps)


class RMSNorm(torch.nn.Module):
    def __init__(self, hidden_size, eps=1e-6, dtype=None, device=None):
        super().__init__()
        self.weight = torch.nn.Parameter(
            torch.ones(hidden_size, dtype=dtype, device=device))
        self.eps = eps

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x):
        return _RMSNormFn.apply(x, self.weight, self.eps)

    def extra_repr(self):
        return f"{self.weight.numel()}, eps={self.eps}"


class FusedLayerNorm(torch.nn.Module):
    def __init__(self, hidden_size, eps=1e-5, bias=True, dtype=None, device=None):
        super().__init__()
        self.weight = torch.nn.Parameter(
            torch.ones(hidden_size, dtype=dtype, device=device))
        self.bias = torch.nn.Parameter(
            torch.zeros(hidden_size, dtype=dtype, device=device)) if bias else None
        self.eps = eps

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)
        if self.bias is not None:
            torch.nn.init.zeros_(self.bias)

    def forward(self, x):
        return _LayerNormFn.apply(x, self.weight, self.bias, self.eps)


def _sk():
    from . import serving_kernels
    return serving_kernels


def scalar_rms_norm(x, gain, eps=1e-6, out_dtype=None, index=None):
    """RMS norm whose gain is ONE number for all coordinates:
    ``x * rsqrt(mean(x^2) + eps) * gain``. Statistics and the product are
    fp32 whatever ``x`` is; the result is rounded once to ``out_dtype``.
    x [T, C] (fp32 residual stream or 16-bit), gain a 0-d/1-element fp32
    tensor. With ``index`` (int64 [R]) the rows ``x[index]`` are normed, the
    gather fused into the kernel (embedding lookup, picking output rows)."""
    out_dtype = out_dtype or x.dtype
    if x.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.scalar_rms_norm(x.contiguous(), gain, eps, out_dtype, index)
    xf = (x if index is None else x[index]).float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) \
        * gain.float().reshape(())
    return y.to(out_dtype)


class ScalarRMSNorm(torch.nn.Module):
    """RMSNorm with a single learned gain (kept fp32)."""

    def __init__(self, eps=1e-6):
        super().__init__()
        self.gain = torch.nn.Parameter(torch.ones(1, dtype=torch.float32),
                                       requires_grad=False)
        self.eps = eps

    def forward(self, x, out_dtype=None, index=None):
        return scalar_rms_norm(x, self.gain, self.eps, out_dtype, index)


def layer_norm_add_(x, y, weight, bias, eps, out_dtype=None):
    """Post-sublayer norm on an fp32 residual stream, in place:
    ``x += (y - mean) / sqrt(var + eps) * weight + bias`` with the statistics
    of each row of ``y`` ([T, C], any float type) in fp32 and ``var`` the mean
    squared deviation. With ``out_dtype`` the same pass also returns the new
    ``x`` rounded to that type (the next sublayer's GEMM operand); otherwise
    it returns ``x``."""
    assert x.dtype == torch.float32 and x.shape == y.shape
    if x.is_cuda and _sk().enabled():
        return _sk().layer_norm_add(x, y, weight, bias, eps, out_dtype)
    yf = y.float()
    mu = yf.mean(-1, keepdim=True)
    d = yf - mu
    var = (d * d).mean(-1, keepdim=True)
    x.add_(d * torch.rsqrt(var + eps) * weight.float() + bias.float())
    return x if out_dtype in (None, torch.float32) else x.to(out_dtype)


def layer_norm_rows(x, weight, bias, eps, out_dtype=None, index=None):
    """Layer norm with weight and bias of the rows ``x[index]`` (all rows
    without ``index``), fp32 statistics, rounded once to ``out_dtype``."""
    out_dtype = out_dtype or x.dtype
    if x.is_cuda and _sk().enabled():
        return _sk().layer_norm_rows(x.contiguous(), weight, bias, eps,
                                     out_dtype, index)
    xf = (x if index is None else x[index]).float()
    mu = xf.mean(-1, keepdim=True)
    d = xf - mu
    var = (d * d).mean(-1, keepdim=True)
    return (d * torch.rsqrt(var + eps) * weight.float()
            + bias.float()).to(out_dtype)


def embed_rows(table, ids, scale, out_dtype=torch.float32, add_table=None,
               add_ids=None):
    """``table[ids] * scale`` in fp32, rounded once to ``out_dtype``. With
    ``add_table`` the rows ``add_table[add_ids]`` (a second table of the same
    width, e.g. a hashed one) are added in fp32 in the same pass."""
    if table.is_cuda and _sk().enabled():
        return _sk().embed_rows(table, ids, scale, out_dtype, add_table,
                                add_ids)
    out = table[ids].float() * scale
    if add_table is not None:
        out = out + add_table[add_ids].float()
    return out.to(out_dtype)


def rms_norm_rows(x, weight, eps, out_dtype=None, index=None, one_plus=False):
    """RMS norm with a weight per coordinate of the rows ``x[index]`` (all
    rows without ``index``): ``x / sqrt(mean(x^2) + eps) * w``, or
    ``* (1 + w)`` with ``one_plus`` (weights stored around zero). fp32
    statistics and product, rounded once to ``out_dtype``. ``x`` may be a
    column slice of a wider tensor."""
    out_dtype = out_dtype or x.dtype
    if x.is_cuda and _sk().enabled():
        if x.stride(-1) != 1:
            x = x.contiguous()
        return _sk().rms_norm_rows(x, weight, eps, out_dtype, index, one_plus)
    xf = (x if index is None else x[index]).float()
    w = weight.float() + 1.0 if one_plus else weight.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
            * w).to(out_dtype)


def gated_add_(x, g1, y1, g2=None, y2=None, norm_weight=None, eps=1e-6,
               out_dtype=None, one_plus=True):
    """Sigmoid-gated residual on an fp32 stream, in place:
    ``x += sigmoid(g1) * y1 (+ sigmoid(g2) * y2)``. ``g*`` are the gates'
    pre-activations ([T, C], may be column slices of a wider projection),
    ``y*`` the sublayers' results; gates, products and the sum are fp32.
    With ``norm_weight`` the same pass also returns the RMS norm of the new
    ``x`` (the next layer's input) in ``out_dtype``; otherwise None."""
    assert x.dtype == torch.float32 and y1.shape == x.shape
    if x.is_cuda and _sk().enabled():
        return _sk().gated_add(x, g1, y1, g2, y2, norm_weight, eps,
                               out_dtype, one_plus)
    d = torch.sigmoid(g1.float()) * y1.float()
    if y2 is not None:
        d = d + torch.sigmoid(g2.float()) * y2.float()
    x.add_(d)
    if norm_weight is None:
        return None
    return rms_norm_rows(x, norm_weight, eps, out_dtype, None, one_plus)


def scaled_add_(x, s1=None, y1=None, s2=None, y2=None, extra=None,
                norm_w1=None, norm_w2=None, eps=1e-6, out_dtype=None):
    """Residual add with a learned factor per column on an fp32 stream, in
    place: ``x += s1 * y1 (+ s2 * y2) (+ extra)``. ``y*`` are sublayer results
    ([T, C], any float type), ``s*`` fp32 [C], ``extra`` fp32 [T, C] added as
    it is; products and the sum are fp32. All three may be absent (the row is
    then only normed). With ``norm_w1`` (and ``norm_w2``) the same pass
    returns the RMS norms ``x / sqrt(mean(x^2) + eps) * w`` of the NEW row
    under each weight in ``out_dtype``: two sublayers that read one row
    through norms of their own share the read and the statistic.
    Returns (h1, h2), None where no weight was given."""
    assert x.dtype == torch.float32
    if x.is_cuda and _sk().enabled():
        return _sk().scaled_add(x, s1, y1, s2, y2, extra, norm_w1, norm_w2,
                                eps, out_dtype)
    if y1 is not None:
        d = s1.float() * y1.float()
        if y2 is not None:
            d = d + s2.float() * y2.float()
        x.add_(d)
    if extra is not None:
        x.add_(extra)
    if norm_w1 is None:
        return None, None
    out_dtype = out_dtype or torch.float32
    n = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    h1 = (n * norm_w1.float()).to(out_dtype)
    h2 = None if norm_w2 is None else (n * norm_w2.float()).to(out_dtype)
    return h1, h2
