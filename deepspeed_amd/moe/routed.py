"""Serving-side mixture of experts: no capacity, no token dropping.

``topk_softmax`` picks each token's ``top`` largest router logits and weights
them by a softmax over the CHOSEN logits only (fp32).
``grouped_sigmoid_topk`` scores experts by ``sigmoid(logit)``, chooses among
the experts of the best few groups by score plus a per-expert correction, and
weights the chosen ones by their uncorrected scores. ``grouped_topk`` is the
general form: sigmoid or full-softmax scores, a group scored by its two best
or its single best choice score, weights optionally renormalised over the
chosen experts and scaled. The last few router outputs may be IDENTITY
experts, which hand the token's input back (times the weight) and have no
weights of their own. ``RoutedExperts`` runs
gated experts (clamped SwiGLU or plain SiLU gating): tokens are grouped by expert, each expert is one pair
of vendor GEMMs on its contiguous group, and a combine kernel sums a token's
weighted expert outputs (plus an optional shared expert scaled by a per-token
sigmoid gate) in fp32. Training-time MoE with capacity and all-to-all lives
in sharded_moe.py.
"""

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops.activations import clamped_swiglu, glu


def _sk():
    from ..ops import serving_kernels
    return serving_kernels


def topk_softmax(logits, top):
    """logits [T, E] fp32 -> (idx [T, top] int64, weight [T, top] fp32)."""
    if logits.is_cuda and _sk().enabled():
        return _sk().topk_softmax(logits.float(), top)
    val, idx = torch.topk(logits.float(), top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def grouped_sigmoid_topk(logits, correction, top, groups=1, keep=1):
    """logits [T, E] fp32, correction [E] fp32. Scores ``s = sigmoid(logits)``;
    choice scores ``c = s + correction``. The E experts form ``groups`` equal
    runs of neighbours; a group's score is the sum of its two largest choice
    scores (its only one when groups hold one expert) and only experts of the
    ``keep`` best groups can be chosen. Returns the ``top`` allowed experts
    with the largest choice scores (idx [T, top] int64) and their weights
    ``s[idx]`` (fp32, not renormalised)."""
    T, E = logits.shape
    assert E % groups == 0 and 1 <= keep <= groups
    assert top <= keep * (E // groups), "more picks than allowed experts"
    if logits.is_cuda and _sk().enabled():
        return _sk().grouped_sigmoid_topk(logits.float(), correction, top,
                                          groups, keep)
    s = torch.sigmoid(logits.float())
    c = s + correction.float()
    if groups > 1:
        per = c.view(T, groups, E // groups)
        gs = per.topk(min(2, E // groups), dim=-1).values.sum(-1)
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(T, groups, dtype=torch.bool, device=c.device)
        allowed.scatter_(1, best, True)
        c = per.masked_fill(~allowed[:, :, None], float("-inf")).view(T, E)
    idx = c.topk(top, dim=-1).indices
    return idx, s.gather(1, idx)


def grouped_topk(logits, correction, top, groups=1, keep=1, score="softmax",
                 group_score="max", renorm=True, scale=1.0):
    """logits [T, E] fp32, correction [E] fp32. Scores ``s`` are
    ``sigmoid(logits)`` or ``softmax(logits)`` over all E; choice scores
    ``c = s + correction``. The E experts form ``groups`` equal runs of
    neighbours scored by the sum of their two largest ``c`` ("top2") or their
    largest ("max"); experts outside the ``keep`` best groups cannot be chosen
    (they count as minus infinity, choice scores may be negative). Returns the
    ``top`` allowed experts with the largest ``c`` (idx [T, top] int64) and
    their weights: ``s[idx]``, with ``renorm`` divided by their sum + 1e-20,
    times ``scale`` (fp32)."""
    T, E = logits.shape
    assert E % groups == 0 and 1 <= keep <= groups
    assert top <= keep * (E // groups), "more picks than allowed experts"
    assert score in ("sigmoid", "softmax") and group_score in ("top2", "max")
    if logits.is_cuda and _sk().enabled():
        return _sk().grouped_topk(logits.float(), correction, top, groups,
                                  keep, score, group_score, renorm, scale)
    z = logits.float()
    s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
    c = s + correction.float()
    if groups > 1:
        per = c.view(T, groups, E // groups)
        n = 1 if group_score == "max" else min(2, E // groups)
        gs = per.topk(n, dim=-1).values.sum(-1)
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(T, groups, dtype=torch.bool, device=c.device)
        allowed.scatter_(1, best, True)
        c = per.masked_fill(~allowed[:, :, None], float("-inf")).view(T, E)
    idx = c.topk(top, dim=-1).indices
    w = s.gather(1, idx)
    if renorm:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return idx, w * scale


def moe_combine(y, inv, weight, shared=None, shared_gate=None):
    """y [N, C] expert outputs; inv [T, top] the row of y that holds each
    (token, choice); weight [T, top] fp32. Returns
    sum_k weight[t, k] * y[inv[t, k]] (+ sigmoid(shared_gate[t]) *
    shared[t]) as [T, C] in y's dtype."""
    if y.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.moe_combine(y, inv, weight, shared, shared_gate)
    out = (y.float()[inv] * weight[..., None]).sum(1)
    if shared is not None:
        out = out + torch.sigmoid(shared_gate.float()) * shared.float()
    return out.to(y.dtype)


class ClampedGLUExpert(nn.Module):
    """down(clamped_swiglu([gate; up] h)) without biases."""

    def __init__(self, width, ff, limit, dtype=torch.float32):
        super().__init__()
        self.limit = float(limit)
        self.w_gu = nn.Parameter(torch.empty(2 * ff, width, dtype=dtype),
                                 requires_grad=False)
        self.w_down = nn.Parameter(torch.empty(width, ff, dtype=dtype),
                                   requires_grad=False)

    def forward(self, h):
        return F.linear(clamped_swiglu(F.linear(h, self.w_gu), self.limit),
                        self.w_down)


class RoutedExperts(nn.Module):
    """``activation``: "clamped_swiglu" (with ``limit``) or a gate name of
    ``ops.activations.glu`` ("silu", "gelu_tanh"). ``router``: "softmax"
    (``topk_softmax`` of logits + ``router_bias``) or "sigmoid_grouped"
    (``grouped_sigmoid_topk`` with ``groups = (count, keep)`` and
    ``router_bias`` as the choice correction) or "softmax_grouped"
    (``grouped_topk``: softmax over all router outputs, groups scored by
    their best choice score, weights renormalised over the chosen experts and
    multiplied by ``route_scale``). ``identity``: the router has that many
    outputs beyond ``experts``; choosing one adds ``weight * h``. Groups are
    formed over experts and identity outputs together."""

    def __init__(self, width, ff, experts, top, limit=0.0, shared_ff=0,
                 shared_limit=0.0, dtype=torch.float32,
                 activation="clamped_swiglu", router="softmax",
                 groups=(1, 1), identity=0, route_scale=1.0):
        super().__init__()
        self.experts, self.top, self.limit = experts, top, float(limit)
        self.activation, self.router_kind = activation, router
        self.groups = (int(groups[0]), int(groups[1]))
        self.identity, self.route_scale = int(identity), float(route_scale)
        if router not in ("softmax", "sigmoid_grouped", "softmax_grouped"):
            raise ValueError(f"unknown router {router!r}")
        if self.identity and router != "softmax_grouped":
            raise ValueError("identity experts come with the softmax_grouped "
                             "router")
        outs = experts + self.identity
        if outs % self.groups[0]:
            raise ValueError("router outputs do not split into equal groups")
        self.router = nn.Parameter(torch.empty(outs, width,
                                               dtype=torch.float32),
                                   requires_grad=False)
        self.router_bias = nn.Parameter(torch.zeros(outs,
                                                    dtype=torch.float32),
                                        requires_grad=False)
        self.w_gu = nn.Parameter(torch.empty(experts, 2 * ff, width,
                                             dtype=dtype), requires_grad=False)
        self.w_down = nn.Parameter(torch.empty(experts, width, ff,
                                               dtype=dtype),
                                   requires_grad=False)
        self.shared = None
        if shared_ff:
            self.shared = ClampedGLUExpert(width, shared_ff, shared_limit,
                                           dtype)
            self.shared_gate = nn.Parameter(torch.empty(1, width, dtype=dtype),
                                            requires_grad=False)

    def _act(self, gu):
        if self.activation == "clamped_swiglu":
            return clamped_swiglu(gu, self.limit)
        return glu(gu, self.activation)

    def route(self, h):
        if self.router_kind == "softmax":
            logits = F.linear(h.float(), self.router.float(),
                              self.router_bias.float())
            return topk_softmax(logits, self.top)
        logits = F.linear(h.float(), self.router.float())
        if self.router_kind == "softmax_grouped":
            return grouped_topk(logits, self.router_bias, self.top,
                                *self.groups, score="softmax",
                                group_score="max", renorm=True,
                                scale=self.route_scale)
        return grouped_sigmoid_topk(logits, self.router_bias, self.top,
                                    *self.groups)

    def forward(self, h, router_input=None):
        """``router_input``: the rows the router reads when they are at hand
        in a wider type than ``h`` (the fp32 normed row beside its 16-bit
        rounding); the experts read ``h``."""
        T = h.shape[0]
        idx, weight = self.route(h if router_input is None else router_input)
        picks = T * self.top
        if picks <= self.DENSE_MAX_PICKS and 2 * picks >= self.experts:
            # decode-sized steps: run every expert on every token as three
            # batched GEMMs (the picks of a few tokens touch most experts'
            # weights anyway) and pick the chosen outputs; no host round trip
            mid = self._act(torch.bmm(h.expand(self.experts, T, -1),
                                      self.w_gu.transpose(1, 2)))
            y = torch.bmm(mid, self.w_down.transpose(1, 2)) \
                .reshape(self.experts * T, -1)
            if self.identity:
                # identity outputs all read the token's own row, kept once
                # after the experts' results: block number ``experts``
                y = torch.cat([y, h], 0)
                idx = idx.clamp(max=self.experts)
            inv = torch.add(self._token_ids(T, h.device), idx, alpha=T)
        else:
            y, inv = self._grouped(h, idx)
        sh = sg = None
        if self.shared is not None:
            sh = self.shared(h)
            sg = F.linear(h, self.shared_gate)
        return moe_combine(y, inv, weight, sh, sg)

    DENSE_MAX_PICKS = 64

    def _token_ids(self, T, device):
        """[T, 1] int64 0..T-1, kept per step size (decode steps repeat)."""
        cache = self.__dict__.setdefault("_ids", {})
        key = (T, str(device))
        if key not in cache:
            if len(cache) > 64:
                cache.clear()
            cache[key] = torch.arange(T, device=device)[:, None]
        return cache[key]

    def _grouped(self, h, idx):
        """Tokens sorted by expert; one pair of GEMMs per expert that has
        tokens. Returns the outputs in sorted order and each pick's place."""
        T = h.shape[0]
        flat = idx.reshape(-1)
        order = torch.argsort(flat, stable=True)
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        counts = torch.bincount(flat, minlength=self.experts
                                + self.identity).tolist()
        xs = h[order // self.top]
        y = torch.empty(T * self.top, h.shape[1], dtype=h.dtype,
                        device=h.device)
        at = 0
        for e, n in enumerate(counts[:self.experts]):
            if n:
                mid = self._act(F.linear(xs[at:at + n], self.w_gu[e]))
                y[at:at + n] = F.linear(mid, self.w_down[e])
                at += n
        if at < y.shape[0]:          # picks of identity outputs: the input
            y[at:] = xs[at:]
        return y, inv.view(T, self.top)
