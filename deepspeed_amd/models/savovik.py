"""Savovik: a decoder-only serving model whose layers run a sequence mixer and
a feed-forward SIDE BY SIDE on one normed input, each scaled by a sigmoid gate
before it joins the fp32 residual stream. Assembled from the framework's
ragged-batch mechanisms.

* layer: ``h = rms(x) * (1 + w)``; ``x += sigmoid(W1 h + b1) * mixer(h)
  + sigmoid(W2 h + b2) * ff(h)`` (ops/norms.py ``gated_add_``, which also hands
  back the next layer's normed input); the gate rows and the feed-forward's up
  rows are one GEMM;
* a layer may run ANOTHER layer's weights (``weights_of``) with a cache stream
  and slot states of its own;
* mixer ``attention``: grouped-query attention over paged K/V rows, rotate-half
  partial rotary with linearly scaled frequencies, values cached at unit RMS,
  scores capped by ``softcap * tanh(s / softcap)``, sliding window
  (ops/window_attention.py);
* mixer ``mamba2``: scalar-decay state-space recurrence with a matrix state per
  head, short convolution on x|B|C, gate before a grouped RMS norm
  (ops/linear_recurrence.py ``ssd_prep``, ``linear_scan``,
  ``gate_group_norm``);
* mixer ``parallel``: two mixers on the same input whose results are added with
  fixed scales: attention with biased projections, per-head query/key norms,
  interleaved rotary with three-band frequency scaling and a mask that confines
  every position to its chunk; and a selective scan with one state vector per
  channel (ops/selective_scan.py). Both read ONE fused input projection and
  feed ONE fused output projection;
* feed-forward: dense, exact (erf) GELU.

The model runs only through a ``PagedStateCache`` step: ``forward`` takes the
flat token list of a ragged batch. Every size and constant comes from the
config.
"""

from dataclasses import dataclass
from typing import List

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..inference.state_cache import PagedStateCache
from ..ops.activations import act_rows
from ..ops.causal_conv import conv_silu_ragged
from ..ops.linear_recurrence import gate_group_norm, linear_scan, ssd_prep
from ..ops.norms import embed_rows, gated_add_, rms_norm_rows
from ..ops.rope import rope_tables
from ..ops.selective_scan import selective_scan
from ..ops.window_attention import attn_prep, window_attention

MIXERS = ("attention", "mamba2", "parallel")


@dataclass
class SavovikConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6
    max_seq_len: int = 1 << 16

    @classmethod
    def from_dict(cls, d: dict) -> "SavovikConfig":
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]),
                  layers=list(d["layers"]), norm_eps=float(d["norm"]["eps"]))
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": "Savovik", "vocab": self.vocab_size,
                "width": self.width, "layers": self.layers,
                "norm": {"eps": self.norm_eps}}

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def owner(self, i: int) -> int:
        """The layer whose tensors layer ``i`` runs."""
        seen = set()
        while self.layers[i].get("weights_of") is not None:
            if i in seen:
                raise ValueError("weights_of forms a cycle")
            seen.add(i)
            i = int(self.layers[i]["weights_of"])
        return i

    def validate(self):
        n = len(self.layers)
        for i, spec in enumerate(self.layers):
            if spec["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {spec['type']!r}")
            src = spec.get("weights_of")
            if src is not None:
                if not 0 <= int(src) < n or int(src) == i:
                    raise ValueError(f"layer {i}: weights_of names no layer")
                o = self.layers[self.owner(i)]
                if o["type"] != spec["type"] or o["mixer"] != spec["mixer"] \
                        or o.get("mlp") != spec.get("mlp"):
                    raise ValueError(f"layer {i}: differs from the layer "
                                     "whose weights it runs")
            mlp = spec.get("mlp")
            if mlp and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown mlp kind "
                                 f"{mlp['kind']!r}")


def _w(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


def _rot_tables(rot, max_seq, device):
    """cos/sin tables [max_seq, dims/2] for a mixer's ``rot`` block: plain
    frequencies ``base^(-2i/dims)``; ``scaling`` with ``original`` is the
    three-band rule, without it every frequency is divided by ``factor``."""
    sc = rot.get("scaling") or {}
    if "original" in sc:
        return rope_tables(int(rot["dims"]), max_seq, float(rot["base"]),
                           device=device, rope_scaling={
                               "factor": float(sc["factor"]),
                               "low_freq_factor": float(sc["low"]),
                               "high_freq_factor": float(sc["high"]),
                               "original_max_position_embeddings":
                                   int(sc["original"])})
    return rope_tables(int(rot["dims"]), max_seq, float(rot["base"]),
                       device=device, scaling=float(sc.get("factor", 1.0)))


class GroupedAttention(nn.Module):
    """Grouped-query attention over paged rows; what differs between its two
    uses is given by flags: projection biases, per-head query/key norms, the
    rotary pairing, unit-RMS values, the score cap and the kind of mask."""

    def __init__(self, m: dict, eps, dtype, *, bias, qk_norm, layout, v_unit,
                 mask):
        super().__init__()
        self.heads = int(m["heads"])
        self.kv_heads = int(m.get("kv_heads", self.heads))
        self.dim, self.vdim = int(m["dim"]), int(m.get("vdim", m["dim"]))
        self.rot = m.get("rot") or {"dims": 0, "base": 10000.0}
        self.rot_dims = int(self.rot.get("dims", 0))
        if self.heads % self.kv_heads or self.rot_dims % 2 or \
                self.rot_dims > self.dim:
            raise ValueError("attention: heads must be a multiple of kv_heads "
                             "and rot.dims even and at most dim")
        self.scale = float(m["scale"])
        self.softcap = float(m.get("softcap") or 0.0)
        size = int((m.get("mask") or {}).get("size", 0))
        self.window = size if mask == "window" else 0
        self.chunk = size if mask == "chunk" else 0
        self.layout = layout
        self.norm = "head" if qk_norm else None
        self.v_unit_eps = eps if v_unit else None
        self.eps = eps
        self.has_bias = bias
        self.n_in = self.heads * self.dim + self.kv_heads * (self.dim
                                                             + self.vdim)
        self.n_out = self.heads * self.vdim
        self.q_norm = _w(self.dim, dtype=torch.float32) if qk_norm else None
        self.k_norm = _w(self.dim, dtype=torch.float32) if qk_norm else None

    @property
    def row_dim(self):
        return self.kv_heads * (self.dim + self.vdim)

    def run(self, proj, cache: PagedStateCache, stream, out=None,
            out_scale=1.0):
        """proj: this step's q|k|v (a column slice is fine). Returns the
        heads' results side by side, before the output projection."""
        b = cache.batch
        cos, sin = _rot_tables(self.rot, cache.max_seq, proj.device) \
            if self.rot_dims else (None, None)
        pool = cache.pools[stream]
        q = attn_prep(proj, b, pool, self.q_norm, self.k_norm, self.eps,
                      self.heads, self.kv_heads, self.dim, self.vdim,
                      self.rot_dims, cos, sin, True, self.norm, self.layout,
                      self.v_unit_eps)
        return window_attention(q, pool, b, self.kv_heads, self.dim,
                                self.vdim, self.scale, self.window, 0, None,
                                self.chunk, self.softcap, out_scale, out)


class AttentionMixer(nn.Module):
    """Mixer 'attention': fused q|k|v projection without biases."""

    def __init__(self, width, m, eps, dtype):
        super().__init__()
        self.att = GroupedAttention(m, eps, dtype, bias=False, qk_norm=False,
                                    layout="half", v_unit=True, mask="window")
        self.w_in = _w(self.att.n_in, width, dtype=dtype)
        self.w_o = _w(width, self.att.n_out, dtype=dtype)

    def row_dims(self):
        return [self.att.row_dim]

    def state_shapes(self, dtype):
        return {}

    def forward(self, h, cache, streams, states):
        o = self.att.run(F.linear(h, self.w_in), cache, streams[0])
        return F.linear(o, self.w_o)


class Mamba2Mixer(nn.Module):
    """Mixer 'mamba2': fused projection z | x | B | C | dt; the recurrence is
    ``linear_scan`` with queries C, keys B, values dt * x and one decay per
    head and token."""

    def __init__(self, width, m, eps, dtype):
        super().__init__()
        self.heads, self.vdim = int(m["heads"]), int(m["vdim"])
        self.state, self.groups = int(m["state"]), int(m.get("groups", 1))
        self.taps = int(m.get("conv", 1))
        self.parts = int(m.get("norm_groups", 1))
        inner = self.heads * self.vdim
        if self.heads % self.groups or inner % self.parts or self.taps < 1:
            raise ValueError("mamba2: heads must be a multiple of groups and "
                             "heads*vdim of norm_groups")
        self.eps = eps
        self.inner = inner
        self.conv_channels = inner + 2 * self.groups * self.state
        self.w_in = _w(inner + self.conv_channels + self.heads, width,
                       dtype=dtype)
        self.conv = _w(self.conv_channels, self.taps, dtype=dtype)
        self.conv_b = _w(self.conv_channels, dtype=torch.float32)
        self.dt_bias = _w(self.heads, dtype=torch.float32)
        self.a_log = _w(self.heads, dtype=torch.float32)
        self.skip = _w(self.heads, dtype=torch.float32)
        self.norm = _w(inner, dtype=torch.float32)
        self.w_o = _w(width, inner, dtype=dtype)

    def row_dims(self):
        return []

    def state_shapes(self, dtype):
        return {"conv": ((max(self.taps - 1, 0), self.conv_channels), dtype),
                "rec": ((self.heads, self.state, self.vdim), torch.float32)}

    def forward(self, h, cache, streams, states):
        b = cache.batch
        proj = F.linear(h, self.w_in)
        Cq, Bk, v, x, decay = ssd_prep(
            proj, b, self.conv, self.conv_b, states["conv"], self.a_log,
            self.dt_bias, self.heads, self.groups, self.state, self.vdim)
        o = linear_scan(Cq, Bk, v, decay, None, states["rec"], b)
        y = gate_group_norm(o, x, self.skip, proj[:, :self.inner], self.norm,
                            self.parts, self.eps, h.dtype)
        return F.linear(y, self.w_o)


class ParallelMixer(nn.Module):
    """Mixer 'parallel': attention inside chunks beside a selective scan.
    ONE input projection ``q | k | v | x | z`` (biases on q, k, v) and ONE
    output projection over ``[left_scale * attention ; right_scale * scan]``
    (the scales are applied where the two results are produced, in fp32)."""

    def __init__(self, width, m, eps, dtype):
        super().__init__()
        self.att = GroupedAttention(m["left"], eps, dtype, bias=True,
                                    qk_norm=True, layout="interleaved",
                                    v_unit=False, mask="chunk")
        r = m["right"]
        self.inner, self.state = int(r["inner"]), int(r["state"])
        self.dt_rank, self.taps = int(r["dt_rank"]), int(r.get("conv", 1))
        self.left_scale = float(m.get("left_scale", 1.0))
        self.right_scale = float(m.get("right_scale", 1.0))
        n_att = self.att.n_in
        self.w_in = _w(n_att + 2 * self.inner, width, dtype=dtype)
        self.b_in = _w(n_att + 2 * self.inner, dtype=dtype)
        self.conv = _w(self.inner, self.taps, dtype=dtype)
        self.conv_b = _w(self.inner, dtype=torch.float32)
        self.w_x = _w(self.dt_rank + 2 * self.state, self.inner, dtype=dtype)
        # the step-size projection runs in fp32 (its few columns cost little)
        self.w_dt = _w(self.inner, self.dt_rank, dtype=torch.float32)
        self.dt_bias = _w(self.inner, dtype=torch.float32)
        self.a_log = _w(self.inner, self.state, dtype=torch.float32)
        self.skip = _w(self.inner, dtype=torch.float32)
        self.w_o = _w(width, self.att.n_out + self.inner, dtype=dtype)

    def row_dims(self):
        return [self.att.row_dim]

    def state_shapes(self, dtype):
        return {"conv": ((max(self.taps - 1, 0), self.inner), dtype),
                "rec": ((self.inner, self.state), torch.float32)}

    def forward(self, h, cache, streams, states):
        b = cache.batch
        T = h.shape[0]
        n_att, n_l, R, N = self.att.n_in, self.att.n_out, self.dt_rank, \
            self.state
        proj = F.linear(h, self.w_in, self.b_in)
        both = torch.empty(T, n_l + self.inner, dtype=h.dtype,
                           device=h.device)
        self.att.run(proj[:, :n_att], cache, streams[0], out=both[:, :n_l],
                     out_scale=self.left_scale)
        x = conv_silu_ragged(proj[:, n_att:n_att + self.inner], self.conv,
                             states["conv"], b, self.conv_b, h.dtype)
        p = F.linear(x, self.w_x)
        dt_pre = F.linear(p[:, :R].float(), self.w_dt)
        selective_scan(x, dt_pre, self.dt_bias, self.a_log, p[:, R:R + N],
                       p[:, R + N:], self.skip, proj[:, n_att + self.inner:],
                       states["rec"], b, h.dtype, self.right_scale,
                       out=both[:, n_l:])
        return F.linear(both, self.w_o)


class SavovikLayer(nn.Module):
    """Weights of one layer: norm, mixer, and ``w_side`` = rows of the mixer's
    gate | the feed-forward's gate | the feed-forward's up projection (one
    GEMM over the normed input; the bias is zero on the up rows)."""

    def __init__(self, cfg: SavovikConfig, spec: dict, dtype):
        super().__init__()
        W, eps, m = cfg.width, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        self.width, self.eps = W, eps
        if self.kind == "attention":
            self.mixer = AttentionMixer(W, m, eps, dtype)
        elif self.kind == "mamba2":
            self.mixer = Mamba2Mixer(W, m, eps, dtype)
        elif self.kind == "parallel":
            self.mixer = ParallelMixer(W, m, eps, dtype)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = _w(W, dtype=torch.float32)
        mlp = spec.get("mlp")
        self.ff = int(mlp["ff"]) if mlp else 0
        n_side = W + (W + self.ff if mlp else 0)
        self.w_side = _w(n_side, W, dtype=dtype)
        self.b_side = _w(n_side, dtype=dtype)
        self.w_down = _w(W, self.ff, dtype=dtype) if mlp else None

    def forward(self, x, h, cache, streams, states, next_norm, dtype):
        """x: fp32 stream, updated in place; h: this layer's normed input.
        Returns the next layer's normed input (None without ``next_norm``)."""
        W = self.width
        side = F.linear(h, self.w_side, self.b_side)
        y = self.mixer(h, cache, streams, states)
        g2 = f = None
        if self.w_down is not None:
            f = F.linear(act_rows(side[:, 2 * W:], "gelu_erf"), self.w_down)
            g2 = side[:, W:2 * W]
        return gated_add_(x, side[:, :W], y, g2, f, next_norm, self.eps, dtype,
                          True)


class SavovikForCausalLM(nn.Module):
    architecture = "Savovik"

    def __init__(self, cfg: SavovikConfig, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        W = cfg.width
        self.embed = _w(cfg.vocab_size, W, dtype=dtype)
        # weights live once per owning layer; ``runs`` lists, per layer of the
        # config, whose weights it runs, its cache streams and its state keys
        self.owners = [cfg.owner(i) for i in range(cfg.num_layers)]
        self.blocks = nn.ModuleDict(
            {str(i): SavovikLayer(cfg, cfg.layers[i], dtype)
             for i in sorted(set(self.owners))})
        self.run_streams, n = [], 0
        for i, o in enumerate(self.owners):
            k = len(self.blocks[str(o)].mixer.row_dims())
            self.run_streams.append(list(range(n, n + k)))
            n += k
        self.final_norm = _w(W, dtype=torch.float32)
        self.head = _w(cfg.vocab_size, W, dtype=dtype)

    def block(self, i):
        """The weights that layer ``i`` of the config runs."""
        return self.blocks[str(self.owners[i])]

    # ------------------------------------------------------------ weights
    def init_random(self, seed=0):
        """Random weights of a useful scale for tests and benchmarks."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("q_norm", "k_norm", "norm"):
                p.data.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf in ("norm1", "final_norm"):
                p.data.copy_(0.1 * torch.randn(p.shape, generator=g))
            elif leaf in ("b_side", "b_in", "conv_b", "dt_bias"):
                p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
            elif leaf == "a_log":
                p.data.copy_(torch.randn(p.shape, generator=g) - 1.0)
            elif leaf == "skip":
                p.data.copy_(torch.randn(p.shape, generator=g))
            elif leaf == "conv":
                p.data.copy_(0.4 * torch.randn(p.shape, generator=g))
            elif name == "embed":
                p.data.copy_(torch.randn(p.shape, generator=g))
            else:
                p.data.copy_(p.shape[-1] ** -0.5
                             * torch.randn(p.shape, generator=g))
        for blk in self.blocks.values():
            if blk.w_down is not None:
                blk.b_side.data[2 * blk.width:] = 0
            if isinstance(blk.mixer, ParallelMixer):
                blk.mixer.b_in.data[blk.mixer.att.n_in:] = 0
        return self

    def load_named_tensors(self, t: dict):
        """Fill the parameters from tensors named as in the checkpoint
        (linear weights [out, in]; 'l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.rg1',
        ...). Rows that share an input are stacked into one projection."""
        def put(p, v):
            if tuple(p.shape) != tuple(v.shape):
                raise ValueError(f"shape {tuple(v.shape)} != "
                                 f"{tuple(p.shape)}")
            p.data.copy_(v.to(p.dtype))

        put(self.embed, t["embed"])
        put(self.final_norm, t["final.norm"])
        put(self.head, t["head"])
        for key, blk in self.blocks.items():
            pre, mp = f"l{key}.", f"l{key}.mix."
            a, W = blk.mixer, blk.width
            put(blk.norm1, t[pre + "norm1"])
            side, bias = [t[pre + "rg1"]], [t[pre + "rg1.b"]]
            if blk.w_down is not None:
                up = t[pre + "mlp.up"]
                side += [t[pre + "rg2"], up]
                bias += [t[pre + "rg2.b"], torch.zeros(up.shape[0],
                                                       dtype=up.dtype)]
                put(blk.w_down, t[pre + "mlp.down"])
            put(blk.w_side, torch.cat(side, 0))
            put(blk.b_side, torch.cat(bias, 0))
            if blk.kind == "attention":
                put(a.w_in, torch.cat([t[mp + n] for n in "qkv"], 0))
                put(a.w_o, t[mp + "o"])
            elif blk.kind == "mamba2":
                put(a.w_in, t[mp + "in"])
                put(a.conv, t[mp + "conv"])
                put(a.conv_b, t[mp + "conv.b"])
                put(a.dt_bias, t[mp + "dt_bias"])
                put(a.a_log, t[mp + "A_log"])
                put(a.skip, t[mp + "D"])
                put(a.norm, t[mp + "norm"])
                put(a.w_o, t[mp + "o"])
            else:
                lp, rp = mp + "left.", mp + "right."
                win = t[rp + "in"]
                put(a.w_in, torch.cat([t[lp + n] for n in "qkv"] + [win], 0))
                put(a.b_in, torch.cat(
                    [t[lp + n + ".b"] for n in "qkv"]
                    + [torch.zeros(win.shape[0], dtype=win.dtype)], 0))
                put(a.att.q_norm, t[lp + "q.norm"])
                put(a.att.k_norm, t[lp + "k.norm"])
                put(a.conv, t[rp + "conv"])
                put(a.conv_b, t[rp + "conv.b"])
                put(a.w_x, t[rp + "x"])
                put(a.w_dt, t[rp + "dt"])
                put(a.dt_bias, t[rp + "dt.b"])
                put(a.a_log, t[rp + "A_log"])
                put(a.skip, t[rp + "D"])
                put(a.w_o, torch.cat([t[lp + "o"], t[rp + "o"]], 1))
        return self

    # -------------------------------------------------------------- cache
    def build_cache(self, max_slots, max_tokens, dtype=None, device=None,
                    block_size=64, **_):
        """One K/V row stream per layer RUN that has attention (a layer that
        runs another's weights still caches its own rows); per request slot
        and layer run the recurrences' states (fp32) and convolution tails."""
        dtype = dtype or self.dtype
        device = device or self.embed.device
        dims, states = [], {}
        for i in range(self.cfg.num_layers):
            mixer = self.block(i).mixer
            dims += mixer.row_dims()
            for k, s in mixer.state_shapes(dtype).items():
                states[f"{k}{i}"] = s
        return PagedStateCache(dims, states, max_slots, max_tokens,
                               block_size=block_size, dtype=dtype,
                               device=device)

    # ------------------------------------------------------------ forward
    @torch.no_grad()
    def forward(self, input_ids, positions=None, kv_cache=None, rows=None,
                taps=None):
        """input_ids: flat [T] tokens of ``kv_cache.batch``. ``rows`` selects
        the flat positions whose logits are returned (default all).
        ``taps`` (a list) receives the stream after every layer."""
        cache = kv_cache
        assert cache is not None and cache.batch is not None, \
            "Savovik runs through a PagedStateCache step"
        ids = input_ids.reshape(-1)
        dt, eps = self.dtype, self.cfg.norm_eps
        x = embed_rows(self.embed, ids, 1.0)
        n = self.cfg.num_layers
        h = rms_norm_rows(x, self.block(0).norm1, eps, dt, None, True) \
            if n else None
        for i in range(n):
            states = {k: cache.states[f"{k}{i}"] for k in ("conv", "rec")
                      if f"{k}{i}" in cache.states}
            nxt = self.block(i + 1).norm1 if i + 1 < n else None
            h = self.block(i)(x, h, cache, self.run_streams[i], states, nxt,
                              dt)
            if taps is not None:
                taps.append(x.clone())
        return F.linear(rms_norm_rows(x, self.final_norm, eps, dt, rows,
                                      True), self.head)

    def num_parameters(self):
        return sum(p.numel() for p in self.parameters())


def build_from_config(cfg: dict, dtype):
    return SavovikForCausalLM(SavovikConfig.from_dict(cfg), dtype)


def savovik_tiny(dtype=torch.float32):
    """A small configuration for tests: every mixer kind, a layer without a
    feed-forward and a layer that runs another layer's weights."""
    att = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.4,
           "softcap": 5.0, "mask": {"size": 9},
           "rot": {"base": 100.0, "dims": 4, "scaling": {"factor": 1.5}}}
    left = {"heads": 2, "kv_heads": 1, "dim": 6, "vdim": 10, "scale": 0.5,
            "mask": {"size": 7},
            "rot": {"base": 50.0, "dims": 4,
                    "scaling": {"factor": 3.0, "low": 1.0, "high": 3.0,
                                "original": 24}}}
    right = {"inner": 20, "state": 5, "dt_rank": 3, "conv": 3}
    m2 = {"heads": 4, "vdim": 5, "state": 6, "groups": 2, "norm_groups": 2,
          "conv": 4}
    ff = {"kind": "dense", "ff": 40}
    cfg = SavovikConfig(
        vocab_size=61, width=24, norm_eps=1e-5,
        layers=[{"type": "mamba2", "mixer": m2, "mlp": ff},
                {"type": "attention", "mixer": att, "mlp": None},
                {"type": "parallel", "mixer": {
                    "left": left, "right": right, "left_scale": 0.8,
                    "right_scale": 1.3}, "mlp": ff},
                {"type": "mamba2", "mixer": m2, "mlp": ff, "weights_of": 0}])
    return SavovikForCausalLM(cfg, dtype)
