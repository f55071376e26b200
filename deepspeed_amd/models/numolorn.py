"""Numolorn: a decoder-only serving model with PARALLEL layers over three
sequence mixers, assembled from the framework's ragged-batch mechanisms.

* embedding: the token's row plus a row of a hashed pair table chosen by
  (previous token, token) (ops/hashed_embedding.py); the previous token is
  carried per request slot;
* a layer reads the fp32 stream ``x`` through two RMS norms of its own and
  adds both sublayers' results, each times a learned factor per column:
  ``x += ls1 * mixer(norm1(x)) + ls2 * ff(norm2(x))`` (ops/norms.py
  ``scaled_add_``: the add of one layer and both norms of the next are one
  pass);
* mixer ``latent_attention``: queries through a normed low-rank latent, keys
  and values from a normed cached latent plus one rotated key part shared by
  the heads (rotate-half pairing), a sink logit per head in the softmax's
  denominator, a sigmoid gate per head (ops/latent_attention.py);
* mixer ``latent_attention_2``: the same cached latent without any rotated
  part, a sliding window, plain softmax, no gate;
* mixer ``channel_delta``: gated delta rule with short convolutions whose
  decay differs per head AND key channel (low-rank projection, softplus step)
  and whose read-out is normed per head and gated by a low-rank sigmoid gate
  (ops/linear_recurrence.py);
* feed-forward: dense SiLU-gated, or routed clamped-SwiGLU experts chosen by a
  softmax router with choice correction, group-limited top-k, renormalised and
  scaled weights and identity experts (moe/routed.py);
* a block of layers may run several times with the same weights; every layer
  RUN has its own cache stream and slot states, and the embedding output is
  added to the stream before each repeated pass;
* the output head is the embedding table, logits times ``logit_scale``.

The model runs only through a ``PagedStateCache`` step: ``forward`` takes the
flat token list of a ragged batch. Every size and constant comes from the
config (two low ranks from tensor shapes).
"""

from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..inference.state_cache import PagedStateCache
from ..moe.routed import RoutedExperts
from ..ops.hashed_embedding import pair_hash_rows
from ..ops.latent_attention import (gate_merge_heads, latent_attention,
                                    latent_prep_parts)
from ..ops.linear_recurrence import (delta_prep, head_norm_gate, linear_scan,
                                     softplus_decay)
from ..ops.norms import embed_rows, rms_norm_rows, scaled_add_
from ..ops.rope import rope_tables
from .lolulorn import GatedMLP

MIXERS = ("latent_attention", "latent_attention_2", "channel_delta")


@dataclass
class NumolornConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    bigram: Optional[dict] = None     # {buckets, mul_prev, mul_cur}
    loop: Optional[dict] = None       # {start, stop, times}
    max_seq_len: int = 1 << 16

    @classmethod
    def from_dict(cls, d: dict) -> "NumolornConfig":
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]),
                  layers=list(d["layers"]), norm_eps=float(d["norm"]["eps"]),
                  logit_scale=float(d.get("logit_scale", 1.0)),
                  bigram=(d.get("embedding") or {}).get("bigram"),
                  loop=d.get("loop"))
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": "Numolorn", "vocab": self.vocab_size,
             "width": self.width, "layers": self.layers,
             "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale}
        if self.bigram:
            d["embedding"] = {"bigram": self.bigram}
        if self.loop:
            d["loop"] = self.loop
        return d

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def validate(self):
        for i, spec in enumerate(self.layers):
            if spec["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {spec['type']!r}")
        if self.loop:
            a, b, t = (int(self.loop[k]) for k in ("start", "stop", "times"))
            if not (0 <= a <= b <= len(self.layers)) or t < 0:
                raise ValueError("loop: need 0 <= start <= stop <= layers "
                                 "and times >= 0")
        if self.bigram and int(self.bigram["buckets"]) < 1:
            raise ValueError("bigram: buckets must be positive")

    def layer_runs(self):
        """[(layer, first layer of a REPEATED pass)] in execution order; the
        index in this list names the run's cache stream and slot states."""
        n = len(self.layers)
        if not self.loop:
            return [(i, False) for i in range(n)]
        a, b, times = (int(self.loop[k]) for k in ("start", "stop", "times"))
        runs = [(i, False) for i in range(a)]
        for t in range(times):
            runs += [(i, t > 0 and i == a) for i in range(a, b)]
        return runs + [(i, False) for i in range(b, n)]


def _w(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


def _pad8(n):
    return (n + 7) // 8 * 8


class LatentAttention(nn.Module):
    """Both latent mixers. With ``q_rank`` the input projection is
    [q latent | kv latent | k_rot | gate logits] and the queries come from the
    normed latent through a second product; without, it is [q | kv latent].
    The per-head key and value up-projections are folded into the query and
    the output (the kernel attends over the cached rows themselves)."""

    def __init__(self, width, m: dict, eps, dtype, positional: bool):
        super().__init__()
        self.heads, self.dim = int(m["heads"]), int(m["dim"])
        self.vdim, self.rank = int(m["vdim"]), int(m["kv_rank"])
        self.rot = int(m.get("rot_dim", 0)) if positional else 0
        rot = m.get("rot") or {}
        self.rot_dims = int(rot.get("dims", self.rot)) if self.rot else 0
        self.rot_base = float(rot.get("base", 10000.0))
        if self.rot_dims % 2 or self.rot_dims > self.rot:
            raise ValueError("latent attention: rot.dims must be even and at "
                             "most rot_dim")
        self.scale = float(m["scale"])
        self.window = int((m.get("mask") or {}).get("size", 0))
        self.q_rank = int(m.get("q_rank", 0)) if positional else 0
        self.has_sink = self.has_gate = positional
        self.eps = eps
        H = self.heads
        nq = H * (self.dim + self.rot)
        first = self.q_rank if self.q_rank else nq
        self.q_cols = first
        rows = first + self.rank + self.rot + (H if self.has_gate else 0)
        self.w_in = _w(_pad8(rows), width, dtype=dtype)
        if self.q_rank:
            self.q_norm = _w(self.q_rank, dtype=torch.float32)
            self.w_uq = _w(nq, self.q_rank, dtype=dtype)
        self.latent_norm = _w(self.rank, dtype=torch.float32)
        self.w_uk = _w(H, self.dim, self.rank, dtype=dtype)    # q_nope -> rank
        self.w_uv = _w(H, self.rank, self.vdim, dtype=dtype)   # rank -> v
        if self.has_sink:
            self.sink = _w(H, dtype=torch.float32)
        self.w_o = _w(width, H * self.vdim, dtype=dtype)

    @property
    def row_dim(self):
        return self.rank + self.rot

    def state_shapes(self, dtype):
        return {}

    def forward(self, h, cache: PagedStateCache, stream, states):
        b = cache.batch
        cos = sin = None
        if self.rot_dims:
            cos, sin = rope_tables(self.rot_dims, cache.max_seq,
                                   self.rot_base, device=h.device)
        pool = cache.pools[stream]
        proj = F.linear(h, self.w_in)
        n0, nkv = self.q_cols, self.rank + self.rot
        if self.q_rank:
            q = F.linear(rms_norm_rows(proj[:, :n0], self.q_norm, self.eps,
                                       h.dtype), self.w_uq)
        else:
            q = proj[:, :n0]
        gate_z = proj[:, n0 + nkv:n0 + nkv + self.heads] if self.has_gate \
            else None
        q_nope, q_rot, gate = latent_prep_parts(
            q, proj[:, n0:n0 + nkv], gate_z, b, pool, self.latent_norm,
            self.eps, self.heads, self.dim, self.rot, self.rank,
            self.rot_dims, cos, sin, layout="half")
        q_lat = torch.bmm(q_nope, self.w_uk)                  # [H, T, rank]
        o_lat = latent_attention(q_lat, q_rot, pool, b, self.rank, self.scale,
                                 window=self.window,
                                 sink=self.sink if self.has_sink else None)
        o = torch.bmm(o_lat, self.w_uv)                       # [H, T, vdim]
        return F.linear(gate_merge_heads(o, gate), self.w_o)


class ChannelDeltaRule(nn.Module):
    """Fused input projection q | k | v | b | a1 | g1 (a1, g1: first factors
    of the low-rank decay and output-gate projections)."""

    def __init__(self, width, m: dict, eps, dtype, a_rank, g_rank):
        super().__init__()
        self.heads = int(m["heads"])
        self.kv_heads = int(m.get("kv_heads", self.heads))
        self.dim, self.vdim = int(m["dim"]), int(m["vdim"])
        self.taps = int(m.get("conv", 1))
        if self.heads % self.kv_heads or self.taps < 1:
            raise ValueError("channel_delta: heads must be a multiple of "
                             "kv_heads")
        self.eps, self.a_rank, self.g_rank = eps, int(a_rank), int(g_rank)
        H = self.heads
        nqk, nv = self.kv_heads * self.dim, H * self.vdim
        self.conv_channels = C = 2 * nqk + nv
        self.b_col, self.a_col = C, C + H
        self.g_col = self.a_col + self.a_rank
        self.w_in = _w(_pad8(self.g_col + self.g_rank), width, dtype=dtype)
        self.conv = _w(C, self.taps, dtype=dtype)
        # the decay's second factor stays fp32: its product feeds the
        # recurrence's exponentials
        self.w_a2 = _w(H * self.dim, self.a_rank, dtype=torch.float32)
        self.dt_bias = _w(H * self.dim, dtype=torch.float32)
        self.a_log = _w(H, dtype=torch.float32)
        self.w_g2 = _w(nv, self.g_rank, dtype=dtype)
        self.norm = _w(self.vdim, dtype=torch.float32)
        self.w_o = _w(width, nv, dtype=dtype)

    row_dim = 0          # nothing cached per token: the state is per slot

    def state_shapes(self, dtype):
        return {"conv": ((max(self.taps - 1, 0), self.conv_channels), dtype),
                "rec": ((self.heads, self.dim, self.vdim), torch.float32)}

    def forward(self, h, cache: PagedStateCache, stream, states):
        b = cache.batch
        proj = F.linear(h, self.w_in)
        q, k, v, beta, _ = delta_prep(
            proj, b, self.conv, states["conv"], None, None, self.kv_heads,
            self.heads, self.dim, self.vdim, beta_col=self.b_col, a_col=-1)
        z = F.linear(proj[:, self.a_col:self.g_col].float(), self.w_a2)
        decay = softplus_decay(z, self.dt_bias, self.a_log, self.heads)
        o = linear_scan(q, k, v, decay, beta, states["rec"], b)
        gate_z = F.linear(proj[:, self.g_col:self.g_col + self.g_rank],
                          self.w_g2)
        y = head_norm_gate(o, self.norm, gate_z, self.eps, h.dtype,
                           act="sigmoid")
        return F.linear(y, self.w_o)


class NumolornLayer(nn.Module):
    def __init__(self, cfg: NumolornConfig, spec: dict, dtype, a_rank=0,
                 g_rank=0):
        super().__init__()
        W, eps, m = cfg.width, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "channel_delta":
            self.mixer = ChannelDeltaRule(W, m, eps, dtype, a_rank, g_rank)
        elif self.kind in MIXERS:
            self.mixer = LatentAttention(
                W, m, eps, dtype, positional=self.kind == "latent_attention")
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = _w(W, dtype=torch.float32)
        self.ls1 = _w(W, dtype=torch.float32)
        mlp = spec.get("mlp")
        self.mlp = self.norm2 = self.ls2 = None
        if mlp:
            self.norm2 = _w(W, dtype=torch.float32)
            self.ls2 = _w(W, dtype=torch.float32)
            if mlp["kind"] == "dense":
                self.mlp = GatedMLP(W, int(mlp["ff"]), "silu", dtype)
            elif mlp["kind"] == "moe":
                r = mlp["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                self.mlp = RoutedExperts(
                    W, int(mlp["expert"]["ff"]), int(r["experts"]),
                    int(r["top"]), float(mlp["expert"]["limit"]), dtype=dtype,
                    activation="clamped_swiglu", router="softmax_grouped",
                    groups=(int(g["count"]), int(g["keep"])),
                    identity=int(r.get("identity", 0)),
                    route_scale=float(r.get("scale", 1.0)))
            else:
                raise ValueError(f"unknown mlp kind {mlp['kind']!r}")

    def forward(self, x, pending, extra, cache, stream, states, dtype, eps):
        """x: fp32 stream. ``pending`` = (ls1, y1, ls2, y2) of the layer run
        before (not yet added) or None; ``extra``: fp32 rows added as they
        are. Adds them, norms the new row under both weights in the same
        pass, and returns this run's own pending results."""
        p = pending or (None, None, None, None)
        h1, h2 = scaled_add_(x, p[0], p[1], p[2], p[3], extra, self.norm1,
                             self.norm2, eps, dtype)
        y1 = self.mixer(h1, cache, stream, states)
        y2 = None
        if isinstance(self.mlp, RoutedExperts) and h2.dtype != torch.float32:
            # the router reads the normed row in fp32, not its 16-bit
            # rounding: a close call is then decided as in 32-bit serving
            y2 = self.mlp(h2, router_input=rms_norm_rows(
                x, self.norm2, eps, torch.float32))
        elif self.mlp is not None:
            y2 = self.mlp(h2)
        return (self.ls1, y1, self.ls2, y2)


class NumolornForCausalLM(nn.Module):
    architecture = "Numolorn"

    def __init__(self, cfg: NumolornConfig, dtype=torch.bfloat16,
                 low_ranks=None):
        """``low_ranks[i] = (a_rank, g_rank)``: ranks of layer i's low-rank
        decay and gate projections (sizes the tensors give, not the config);
        default ``mixer.a_rank`` / ``mixer.g_rank`` or ``dim // 2``."""
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        W = cfg.width
        low_ranks = low_ranks or {}
        self.embed = _w(cfg.vocab_size, W, dtype=dtype)
        self.bigram = None
        if cfg.bigram:
            self.bigram = _w(int(cfg.bigram["buckets"]) + 1, W, dtype=dtype)
        layers = []
        for i, s in enumerate(cfg.layers):
            m = s["mixer"]
            d = max(1, int(m.get("dim", 2)) // 2)
            ar, gr = low_ranks.get(i, (int(m.get("a_rank", d)),
                                       int(m.get("g_rank", d))))
            layers.append(NumolornLayer(cfg, s, dtype, ar, gr))
        self.layers = nn.ModuleList(layers)
        self.runs = cfg.layer_runs()
        # cache stream of every layer run that caches rows
        self.stream_of, n = {}, 0
        for r, (i, _) in enumerate(self.runs):
            if self.layers[i].mixer.row_dim:
                self.stream_of[r] = n
                n += 1
        self.final_norm = _w(W, dtype=torch.float32)

    # ------------------------------------------------------------ weights
    def init_random(self, seed=0):
        """Random weights of a useful scale for tests and benchmarks."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            rnd = torch.randn(p.shape, generator=g)
            if leaf in ("norm1", "norm2", "final_norm", "q_norm",
                        "latent_norm", "norm"):
                p.data.copy_(1 + 0.1 * rnd)
            elif leaf in ("ls1", "ls2"):
                p.data.copy_(0.6 + 0.2 * rnd)
            elif leaf in ("router_bias",):
                p.data.copy_(0.05 * rnd)
            elif leaf in ("dt_bias", "sink"):
                p.data.copy_(0.5 * rnd)
            elif leaf == "a_log":
                p.data.copy_(rnd - 1.0)
            elif leaf == "conv":
                p.data.copy_(0.4 * rnd)
            elif name in ("embed", "bigram"):
                p.data.copy_(0.7 * rnd)
            else:
                p.data.copy_(p.shape[-1] ** -0.5 * rnd)
        return self

    def load_named_tensors(self, t: dict):
        """Fill the parameters from tensors named as in the checkpoint
        (linear weights [out, in]; 'l<i>.mix.*', 'l<i>.mlp.*', ...)."""
        def put(p, v):
            if tuple(p.shape) != tuple(v.shape):
                raise ValueError(f"shape {tuple(v.shape)} != "
                                 f"{tuple(p.shape)}")
            p.data.copy_(v.to(p.dtype))

        def put_rows(p, parts):
            """Stacked rows; the parameter may be padded with zero rows."""
            v = torch.cat(parts, 0)
            if v.shape[0] > p.shape[0] or v.shape[1:] != p.shape[1:]:
                raise ValueError(f"rows {tuple(v.shape)} do not fit "
                                 f"{tuple(p.shape)}")
            p.data.zero_()
            p.data[:v.shape[0]].copy_(v.to(p.dtype))

        put(self.embed, t["embed"])
        if self.bigram is not None:
            put(self.bigram, t["bigram"])
        put(self.final_norm, t["final.norm"])
        for i, layer in enumerate(self.layers):
            pre, mp = f"l{i}.", f"l{i}.mix."
            a = layer.mixer
            put(layer.norm1, t[pre + "norm1"])
            put(layer.ls1, t[pre + "ls1"])
            if layer.kind == "channel_delta":
                put_rows(a.w_in, [t[mp + n] for n in
                                  ("q", "k", "v", "b", "a1", "g1")])
                put(a.conv, torch.cat([t[mp + n + ".conv"] for n in "qkv"], 0))
                put(a.w_a2, t[mp + "a2"])
                put(a.dt_bias, t[mp + "dt_bias"])
                put(a.a_log, t[mp + "A_log"])
                put(a.w_g2, t[mp + "g2"])
                put(a.norm, t[mp + "norm"])
            else:
                if a.q_rank:
                    put_rows(a.w_in, [t[mp + "dq"], t[mp + "dkv"],
                                      t[mp + "g"]])
                    put(a.q_norm, t[mp + "dq.norm"])
                    put(a.w_uq, t[mp + "uq"])
                else:
                    put_rows(a.w_in, [t[mp + "q"], t[mp + "dkv"]]
                             + ([t[mp + "g"]] if a.has_gate else []))
                if a.has_sink:
                    put(a.sink, t[mp + "sink"])
                put(a.latent_norm, t[mp + "dkv.norm"])
                put(a.w_uk, t[mp + "uk"].reshape(a.heads, a.dim, a.rank))
                put(a.w_uv, t[mp + "uv"].reshape(a.heads, a.vdim, a.rank)
                    .transpose(1, 2))
            put(a.w_o, t[mp + "o"])
            m = layer.mlp
            if m is None:
                continue
            put(layer.norm2, t[pre + "norm2"])
            put(layer.ls2, t[pre + "ls2"])
            fp = pre + "mlp."
            if isinstance(m, GatedMLP):
                put(m.w_gu, torch.cat([t[fp + "gate"], t[fp + "up"]], 0))
                put(m.w_down, t[fp + "down"])
            else:
                put(m.router, t[fp + "router"])
                put(m.router_bias, t[fp + "correction"])
                put(m.w_gu, torch.stack(
                    [torch.cat([t[f"{fp}e{e}.gate"], t[f"{fp}e{e}.up"]], 0)
                     for e in range(m.experts)]))
                put(m.w_down, torch.stack([t[f"{fp}e{e}.down"]
                                           for e in range(m.experts)]))
        return self

    def named_tensors(self):
        """The parameters under their checkpoint names (the inverse of
        ``load_named_tensors``), for writing a model folder."""
        t = {"embed": self.embed, "final.norm": self.final_norm}
        if self.bigram is not None:
            t["bigram"] = self.bigram
        for i, layer in enumerate(self.layers):
            pre, mp = f"l{i}.", f"l{i}.mix."
            a = layer.mixer
            t[pre + "norm1"], t[pre + "ls1"] = layer.norm1, layer.ls1
            if layer.kind == "channel_delta":
                nqk, nv, H = a.kv_heads * a.dim, a.heads * a.vdim, a.heads
                cuts = [nqk, nqk, nv, H, a.a_rank, a.g_rank]
                at = 0
                for n, c in zip(("q", "k", "v", "b", "a1", "g1"), cuts):
                    t[mp + n] = a.w_in[at:at + c]
                    at += c
                at = 0
                for n, c in zip("qkv", cuts[:3]):
                    t[mp + n + ".conv"] = a.conv[at:at + c]
                    at += c
                t[mp + "a2"], t[mp + "dt_bias"] = a.w_a2, a.dt_bias
                t[mp + "A_log"], t[mp + "g2"] = a.a_log, a.w_g2
                t[mp + "norm"] = a.norm
            else:
                n0, nkv = a.q_cols, a.rank + a.rot
                if a.q_rank:
                    t[mp + "dq"], t[mp + "dq.norm"] = a.w_in[:n0], a.q_norm
                    t[mp + "uq"] = a.w_uq
                else:
                    t[mp + "q"] = a.w_in[:n0]
                t[mp + "dkv"] = a.w_in[n0:n0 + nkv]
                if a.has_gate:
                    t[mp + "g"] = a.w_in[n0 + nkv:n0 + nkv + a.heads]
                if a.has_sink:
                    t[mp + "sink"] = a.sink
                t[mp + "dkv.norm"] = a.latent_norm
                t[mp + "uk"] = a.w_uk.reshape(a.heads * a.dim, a.rank)
                t[mp + "uv"] = a.w_uv.transpose(1, 2) \
                    .reshape(a.heads * a.vdim, a.rank)
            t[mp + "o"] = a.w_o
            m = layer.mlp
            if m is None:
                continue
            t[pre + "norm2"], t[pre + "ls2"] = layer.norm2, layer.ls2
            fp = pre + "mlp."
            if isinstance(m, GatedMLP):
                ff = m.w_gu.shape[0] // 2
                t[fp + "gate"], t[fp + "up"] = m.w_gu[:ff], m.w_gu[ff:]
                t[fp + "down"] = m.w_down
            else:
                ff = m.w_gu.shape[1] // 2
                t[fp + "router"], t[fp + "correction"] = m.router, \
                    m.router_bias
                for e in range(m.experts):
                    t[f"{fp}e{e}.gate"] = m.w_gu[e, :ff]
                    t[f"{fp}e{e}.up"] = m.w_gu[e, ff:]
                    t[f"{fp}e{e}.down"] = m.w_down[e]
        return {k: v.detach().contiguous() for k, v in t.items()}

    # -------------------------------------------------------------- cache
    def build_cache(self, max_slots, max_tokens, dtype=None, device=None,
                    block_size=64, **_):
        """One latent row stream per attention layer RUN; per request slot
        and recurrent layer run the matrix state (fp32) and the convolution
        tail; per slot the last token fed (the hashed embedding's state)."""
        dtype = dtype or self.dtype
        device = device or self.embed.device
        dims = [self.layers[self.runs[r][0]].mixer.row_dim
                for r in sorted(self.stream_of, key=self.stream_of.get)]
        states = {}
        for r, (i, _) in enumerate(self.runs):
            for k, s in self.layers[i].mixer.state_shapes(dtype).items():
                states[f"{k}{r}"] = s
        if self.bigram is not None:
            states["prev"] = ((), torch.int64)
        return PagedStateCache(dims, states, max_slots, max_tokens,
                               block_size=block_size, dtype=dtype,
                               device=device)

    # ------------------------------------------------------------ forward
    @torch.no_grad()
    def forward(self, input_ids, positions=None, kv_cache=None, rows=None,
                taps=None):
        """input_ids: flat [T] tokens of ``kv_cache.batch``. ``rows`` selects
        the flat positions whose logits are returned (default all).
        ``taps`` (a list) receives the stream after every layer run."""
        cache = kv_cache
        assert cache is not None and cache.batch is not None, \
            "Numolorn runs through a PagedStateCache step"
        ids = input_ids.reshape(-1)
        dt, eps = self.dtype, self.cfg.norm_eps
        if self.bigram is not None:
            bg = self.cfg.bigram
            pair = pair_hash_rows(ids, cache.batch, cache.states["prev"],
                                  int(bg["mul_prev"]), int(bg["mul_cur"]),
                                  int(bg["buckets"]))
            x = embed_rows(self.embed, ids, 1.0, add_table=self.bigram,
                           add_ids=pair)
        else:
            x = embed_rows(self.embed, ids, 1.0)
        x0 = x.clone() if any(again for _, again in self.runs) else None
        pending = None
        for r, (i, again) in enumerate(self.runs):
            states = {k: cache.states[f"{k}{r}"] for k in ("conv", "rec")
                      if f"{k}{r}" in cache.states}
            pending = self.layers[i](x, pending, x0 if again else None, cache,
                                     self.stream_of.get(r), states, dt, eps)
            if taps is not None:
                scaled_add_(x, *pending)
                pending = None
                taps.append(x.clone())
        if pending is not None:
            scaled_add_(x, *pending)
        return F.linear(rms_norm_rows(x, self._final_weight(), eps, dt, rows),
                        self.embed)

    def _final_weight(self):
        """logits = table . (norm(x) * w) * scale: the scale rides on the
        norm's weight, so no pass over [rows, vocab] is needed for it. The
        product is kept until the weight changes."""
        w = self.final_norm
        if self.cfg.logit_scale == 1.0:
            return w
        kept = self.__dict__.get("_scaled_final")
        if kept is None or kept[0] != (w._version, w.device, w.data_ptr()):
            kept = ((w._version, w.device, w.data_ptr()),
                    w.detach() * self.cfg.logit_scale)
            self.__dict__["_scaled_final"] = kept
        return kept[1]

    def num_parameters(self):
        return sum(p.numel() for p in self.parameters())


def build_from_config(cfg: dict, dtype, tensors=None):
    """Registry entry. The ranks of the recurrent mixer's low-rank decay and
    gate projections are sizes that only the tensors give."""
    ranks = {}
    for i, spec in enumerate(cfg["layers"]):
        if spec["type"] == "channel_delta" and tensors is not None and \
                f"l{i}.mix.a1" in tensors:
            ranks[i] = (int(tensors[f"l{i}.mix.a1"].shape[0]),
                        int(tensors[f"l{i}.mix.g1"].shape[0]))
    return NumolornForCausalLM(NumolornConfig.from_dict(cfg), dtype, ranks)


def numolorn_tiny(dtype=torch.float32):
    """A small configuration for tests: every mixer kind, a dense and a
    routed feed-forward with identity experts, a layer without feed-forward,
    a looped block."""
    la = {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 12,
          "q_rank": 10, "rot": {"base": 100.0, "dims": 4}, "scale": 0.3}
    lw = {"heads": 2, "dim": 6, "vdim": 5, "kv_rank": 9, "scale": 0.4,
          "mask": {"size": 7}}
    cd = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "conv": 3,
          "a_rank": 4, "g_rank": 3}
    moe = {"kind": "moe", "expert": {"ff": 12, "limit": 1.2},
           "router": {"experts": 5, "top": 2, "identity": 1, "scale": 1.3,
                      "groups": {"count": 3, "keep": 2}}}
    cfg = NumolornConfig(
        vocab_size=59, width=24, norm_eps=1e-5, logit_scale=0.7,
        bigram={"buckets": 37, "mul_prev": 5, "mul_cur": 11},
        loop={"start": 1, "stop": 3, "times": 2},
        layers=[{"type": "latent_attention_2", "mixer": lw,
                 "mlp": {"kind": "dense", "ff": 40}},
                {"type": "channel_delta", "mixer": cd, "mlp": moe},
                {"type": "latent_attention", "mixer": la, "mlp": None},
                {"type": "latent_attention", "mixer": la, "mlp": moe}])
    return NumolornForCausalLM(cfg, dtype)
