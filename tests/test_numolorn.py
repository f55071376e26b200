"""Numolorn through the serving path (registry -> ContinuousBatcher ->
PagedStateCache -> ops) against the plain oracle in numolorn_oracle.py.

Every test makes its own small configuration and random tensors under the
checkpoint's names; the same tensors feed the oracle (float64) and
``load_named_tensors``. The device is the GPU when there is one (tests marked
``gpu`` then run the HIP kernels), the CPU otherwise.
"""

import json
import math
import os

import pytest
import torch

from tests import numolorn_oracle as O
from deepspeed_amd.inference.ragged import ContinuousBatcher, Request
from deepspeed_amd.inference.state_cache import PagedStateCache
from deepspeed_amd.models import build_model, load_pretrained

DEV = "cuda" if torch.cuda.is_available() else "cpu"


# ------------------------------------------------------- configurations
def la(heads=3, dim=8, rot=4, vdim=6, rank=12, q_rank=10, dims=None,
       base=100.0, scale=0.3):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot,
                      "vdim": vdim, "kv_rank": rank, "q_rank": q_rank,
                      "rot": {"base": base, "dims": rot if dims is None
                              else dims}, "scale": scale}}


def lw(heads=2, dim=6, vdim=5, rank=9, win=7, scale=0.4):
    return {"type": "latent_attention_2",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim,
                      "kv_rank": rank, "scale": scale,
                      "mask": {"size": win}}}


def cd(heads=4, kv=2, dim=6, vdim=5, conv=3, a_rank=4, g_rank=3):
    """``_ranks`` is read by ``tensors`` only (the model takes both ranks
    from the tensors' shapes)."""
    return {"type": "channel_delta",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim,
                      "vdim": vdim, "conv": conv},
            "_ranks": (a_rank, g_rank)}


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(ff=12, limit=1.2, experts=5, top=2, identity=1, scale=1.3, count=3,
        keep=2):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "identity": identity,
                       "scale": scale,
                       "groups": {"count": count, "keep": keep}}}


def config(layers, width=24, vocab=41, eps=1e-5, loop=None, logit_scale=0.7,
           bigram=(37, 5, 11)):
    """layers: (mixer entry, mlp or None) pairs."""
    cfg = {"architecture": "Numolorn", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "logit_scale": logit_scale,
           "embedding": {"bigram": {"buckets": bigram[0],
                                    "mul_prev": bigram[1],
                                    "mul_cur": bigram[2]}},
           "layers": [{**mix, "mlp": mlp} for mix, mlp in layers]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tensors(cfg, seed=0):
    """Random tensors of a useful scale under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rn(*shape, s=1.0):
        return torch.randn(*shape, generator=g) * s

    def lin(o, i):
        return rn(o, i, s=i ** -0.5)

    t = {"embed": rn(cfg["vocab"], W, s=0.7),
         "bigram": rn(cfg["embedding"]["bigram"]["buckets"] + 1, W, s=0.7),
         "final.norm": 1 + rn(W, s=0.1)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        t[p + "norm1"], t[p + "ls1"] = 1 + rn(W, s=0.1), 0.6 + rn(W, s=0.2)
        q = p + "mix."
        if spec["type"] == "channel_delta":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            ar, gr = spec["_ranks"]
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
                t[q + n] = lin(rows, W)
                t[q + n + ".conv"] = rn(rows, m["conv"], s=0.5)
            t[q + "b"] = lin(H, W)
            t[q + "A_log"] = rn(H) - 1.0
            t[q + "norm"] = 1 + rn(dv, s=0.1)
            t[q + "a1"], t[q + "a2"] = lin(ar, W), lin(H * d, ar)
            t[q + "dt_bias"] = rn(H * d, s=0.5)
            t[q + "g1"], t[q + "g2"] = lin(gr, W), lin(H * dv, gr)
            t[q + "o"] = lin(W, H * dv)
        else:
            H, d, dv, r = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
            rot = m.get("rot_dim", 0)
            if spec["type"] == "latent_attention":
                t[q + "dq"] = lin(m["q_rank"], W)
                t[q + "dq.norm"] = 1 + rn(m["q_rank"], s=0.1)
                t[q + "uq"] = lin(H * (d + rot), m["q_rank"])
                t[q + "sink"] = rn(H, s=0.7)
                t[q + "g"] = lin(H, W)
            else:
                t[q + "q"] = lin(H * d, W)
            t[q + "dkv"] = lin(r + rot, W)
            t[q + "dkv.norm"] = 1 + rn(r, s=0.1)
            t[q + "uk"], t[q + "uv"] = lin(H * d, r), lin(H * dv, r)
            t[q + "o"] = lin(W, H * dv)
        mlp = spec["mlp"]
        if not mlp:
            continue
        t[p + "norm2"], t[p + "ls2"] = 1 + rn(W, s=0.1), 0.6 + rn(W, s=0.2)
        f = p + "mlp."
        if mlp["kind"] == "dense":
            t[f + "gate"], t[f + "up"] = lin(mlp["ff"], W), lin(mlp["ff"], W)
            t[f + "down"] = lin(W, mlp["ff"])
        else:
            r, ff = mlp["router"], mlp["expert"]["ff"]
            n = r["experts"] + r["identity"]
            t[f + "router"] = rn(n, W, s=2.0 * W ** -0.5)
            # corrections on both sides of zero: choice scores go negative
            t[f + "correction"] = rn(n, s=0.2)
            for e in range(r["experts"]):
                t[f"{f}e{e}.gate"] = lin(ff, W) * 2
                t[f"{f}e{e}.up"] = lin(ff, W) * 2
                t[f"{f}e{e}.down"] = lin(W, ff)
    return t


def strip(cfg):
    """The configuration as a checkpoint folder holds it."""
    return {**cfg, "layers": [{k: v for k, v in s.items() if k != "_ranks"}
                              for s in cfg["layers"]]}


BASE = config([(lw(), dense(40)),
               (cd(), moe()),
               (la(), None),
               (la(heads=2, dim=4, rot=6, vdim=8, rank=10, q_rank=5, dims=4),
                moe(experts=4, top=3, identity=2, count=2, keep=1)),
               (cd(heads=2, kv=2, dim=8, vdim=4, conv=2, a_rank=2, g_rank=5),
                dense(16))],
              loop=(1, 3, 2))


class Served:
    """A configuration loaded into the framework plus its oracle weights."""

    def __init__(self, cfg, seed=0, dtype=torch.float32, slots=4,
                 max_tokens=512, block=16, t=None):
        self.cfg = strip(cfg)
        self.t = t or tensors(cfg, seed)
        if dtype == torch.bfloat16:
            # the oracle gets the weights as 16-bit serving holds them, so
            # what is measured is the arithmetic, not a router's close call
            self.t = {k: v.bfloat16().float() for k, v in self.t.items()}
        self.w64 = {k: v.double() for k, v in self.t.items()}
        self.model = build_model(self.cfg, dtype, self.t) \
            .load_named_tensors(self.t).to(DEV).eval()
        self.model.build_cache = self._cache(self.model.build_cache, block)
        self.batcher = ContinuousBatcher(self.model, max_slots=slots,
                                         dtype=dtype, device=torch.device(DEV),
                                         max_tokens=max_tokens)
        self.n = 0

    @staticmethod
    def _cache(build, block):
        return lambda *a, **k: build(*a, **{**k, "block_size": block})

    def oracle(self, tokens, streams=None):
        return O.forward(list(tokens), self.w64, self.cfg, streams=streams)

    def run(self, tokens, cuts):
        """One request fed in portions ``cuts``; logits of every position."""
        self.n += 1
        req = self.batcher.open("q%d" % self.n)
        out, at = [], 0
        for c in cuts:
            out.append(self.batcher.feed([(req, tokens[at:at + c])]).double()
                       .cpu())
            at += c
        assert at == len(tokens)
        self.batcher.close(req)
        return torch.cat(out)


def toks(n, vocab=41, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, want, tol=2e-4):
    scale = want.std().item()
    err = (got - want).abs().max().item() / scale
    assert err < tol, "relative error %.3g" % err


def close_rms(got, want, tol, flips=0.0):
    """16-bit runs: root-mean-square error per position, against the spread.
    ``flips``: the share of positions that may exceed ``tol`` because 16-bit
    rounding turned a router's close call (another expert, a visibly
    different row); they stay bounded all the same."""
    err = ((got - want) ** 2).mean(-1).sqrt() / want.std().item()
    over = (err >= tol).sum().item()
    assert over <= flips * err.numel(), \
        "%d of %d positions over %.3g, worst %.3g" % (over, err.numel(), tol,
                                                      err.max().item())
    assert err.max().item() < (0.6 if flips else tol)


def one_step_cache(row_dims, states, held, counts, block=8, tokens=512,
                   dtype=torch.float32):
    """A cache whose slots already hold ``held`` tokens, with a step of
    ``counts`` new ones begun."""
    cache = PagedStateCache(row_dims, states, len(held), tokens,
                            block_size=block, device=DEV, dtype=dtype)
    for slot, n in enumerate(held):
        cache.reset_slot(slot)
        cache.lens[slot] = n
    return cache, cache.begin_ragged(list(range(len(held))), counts)


def pool_index(cache, slot, positions):
    bs, tab = cache.block_size, cache.block_table[slot]
    return torch.tensor([tab[p // bs] * bs + p % bs for p in positions]).to(DEV)


# ------------------------------------------------------ mechanisms alone
def test_pair_hash_rows_carry_the_previous_token_across_steps_and_slots():
    from deepspeed_amd.ops.hashed_embedding import pair_hash_rows
    cfg = {"embedding": {"bigram": {"buckets": 13, "mul_prev": 7,
                                    "mul_cur": 3}}}
    cache = PagedStateCache([], {"prev": ((), torch.int64)}, 3, 256,
                            block_size=8, device=DEV)
    seqs = {0: toks(11, seed=1), 2: toks(6, seed=2)}
    plan = [{0: 4, 2: 1}, {2: 2}, {0: 1, 2: 3}, {0: 6}]
    for s in seqs:
        cache.reset_slot(s)
    at, got = {0: 0, 2: 0}, {0: [], 2: []}
    for step in plan:
        b = cache.begin_ragged(list(step), list(step.values()))
        ids = torch.tensor([x for s, n in step.items()
                            for x in seqs[s][at[s]:at[s] + n]]).to(DEV)
        rows = pair_hash_rows(ids, b, cache.states["prev"], 7, 3, 13).cpu()
        cache.end_step()
        o = 0
        for s, n in step.items():
            got[s] += rows[o:o + n].tolist()
            o += n
            at[s] += n
    for s, seq in seqs.items():
        want = [13] + [(seq[i - 1] * 7 + seq[i] * 3) % 13
                       for i in range(1, len(seq))]
        assert got[s] == want
    # a slot handed out again starts with the table's last row
    cache.reset_slot(0)
    b = cache.begin_ragged([0], [2])
    rows = pair_hash_rows(torch.tensor([5, 6]).to(DEV), b,
                          cache.states["prev"], 7, 3, 13).cpu().tolist()
    assert rows == [13, (5 * 7 + 6 * 3) % 13]
    # the oracle's embedding is the sum of both rows
    w = {"embed": torch.randn(41, 4).double(),
         "bigram": torch.randn(14, 4).double()}
    e = O.embedding(seqs[0], w, cfg)
    assert torch.equal(e[0], w["embed"][seqs[0][0]] + w["bigram"][13])


def test_embedding_sum_of_two_tables():
    from deepspeed_amd.ops.norms import embed_rows
    a, b = torch.randn(9, 16).to(DEV), torch.randn(5, 16).to(DEV)
    i, j = torch.tensor([3, 8, 0]).to(DEV), torch.tensor([4, 4, 1]).to(DEV)
    got = embed_rows(a, i, 1.0, add_table=b, add_ids=j)
    assert got.dtype == torch.float32
    assert torch.allclose(got, a[i] + b[j])


@pytest.mark.parametrize("two,extra", [(False, False), (True, False),
                                       (True, True)])
def test_scaled_residual_and_the_two_norms_it_hands_on(two, extra):
    from deepspeed_amd.ops.norms import scaled_add_
    T, C, eps = 5, 24, 1e-5
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, C, generator=g).to(DEV)
    y1, y2 = torch.randn(T, C, generator=g).to(DEV), \
        torch.randn(T, C, generator=g).to(DEV)
    s1, s2 = torch.randn(C, generator=g).to(DEV), \
        torch.randn(C, generator=g).to(DEV)
    w1, w2 = torch.randn(C, generator=g).to(DEV), \
        torch.randn(C, generator=g).to(DEV)
    ex = torch.randn(T, C, generator=g).to(DEV) if extra else None
    want = x.double() + s1.double() * y1.double()
    if two:
        want = want + s2.double() * y2.double()
    if extra:
        want = want + ex.double()
    n = O.rms(want, eps)
    h1, h2 = scaled_add_(x, s1, y1, s2 if two else None, y2 if two else None,
                         ex, w1, w2 if two else None, eps)
    close(x.double().cpu(), want.cpu(), 1e-6)
    close(h1.double().cpu(), (n * w1.double()).cpu(), 1e-5)
    if two:
        close(h2.double().cpu(), (n * w2.double()).cpu(), 1e-5)
    else:
        assert h2 is None
    # nothing to add: the row is only normed
    before = x.clone()
    h1, _ = scaled_add_(x, norm_w1=w1, eps=eps)
    assert torch.equal(x, before)
    close(h1.double().cpu(), (O.rms(x.double(), eps) * w1.double()).cpu(), 1e-5)


@pytest.mark.parametrize("rot,dims", [(4, 4), (6, 4), (8, 2)])
def test_latent_prologue_rotates_halves_and_norms_the_latent(rot, dims):
    """Rows of the pool and rotated queries against the oracle's rotation at
    positions that a second step starts in the middle of."""
    from deepspeed_amd.ops.latent_attention import latent_prep_parts
    from deepspeed_amd.ops.rope import rope_tables
    H, d, rank, base, eps = 2, 3, 5, 50.0, 1e-5
    held, cnt = 9, 6
    cache, b = one_step_cache([rank + rot], {}, [held], [cnt])
    g = torch.Generator().manual_seed(rot * 10 + dims)
    q = torch.randn(cnt, H * (d + rot), generator=g).to(DEV)
    kv = torch.randn(cnt, rank + rot, generator=g).to(DEV)
    gz = torch.randn(cnt, H, generator=g).to(DEV)
    nw = torch.randn(rank, generator=g).to(DEV)
    cos, sin = rope_tables(dims, cache.max_seq, base, device=DEV)
    wide = torch.cat([q, kv, gz], -1)          # operands as column slices
    nq = H * (d + rot)
    q_nope, q_rot, gate = latent_prep_parts(
        wide[:, :nq], wide[:, nq:nq + rank + rot], wide[:, nq + rank + rot:],
        b, cache.pools[0], nw, eps, H, d, rot, rank, dims, cos, sin,
        layout="half")
    full = torch.zeros(held + cnt, H, rot, dtype=torch.float64)
    full[held:] = q.double().cpu().view(cnt, H, d + rot)[..., d:]
    want_q = O.rotate_half(full, dims, base)[held:]
    close(q_rot.double().cpu(), want_q, 1e-5)
    fk = torch.zeros(held + cnt, 1, rot, dtype=torch.float64)
    fk[held:, 0] = kv.double().cpu()[:, rank:]
    want_k = O.rotate_half(fk, dims, base)[held:, 0]
    rows = cache.pools[0].view(-1, rank + rot)[
        pool_index(cache, 0, range(held, held + cnt))].double().cpu()
    close(rows[:, rank:], want_k, 1e-5)
    close(rows[:, :rank], O.rms(kv.double().cpu()[:, :rank], eps)
          * nw.double().cpu(), 1e-5)
    close(gate.double().cpu(), O.sigmoid(gz.double().cpu()), 1e-5)
    close(q_nope.double().cpu(),
          q.double().cpu().view(cnt, H, d + rot)[..., :d].transpose(0, 1),
          1e-6)


def _crafted_latent(held, count, target, window=0, sink=None, rank=8, H=2,
                    block=8, dtype=torch.float32, big=40.0):
    """Rows whose first coordinate is 1 at ``target`` and 0 elsewhere (small
    noise on the rest), queries that score ``big`` on that coordinate: a
    query that sees the target returns the target's row, one that does not
    returns a blend of the noise rows. Returns out [H, count, rank], rows."""
    from deepspeed_amd.ops.latent_attention import latent_attention
    n = held + count
    cache, b = one_step_cache([rank], {}, [3, held], [1, count], block=block,
                              tokens=4096, dtype=dtype)
    g = torch.Generator().manual_seed(target + 7 * n)
    rows = 0.05 * torch.randn(n, rank, generator=g)
    rows[:, 0] = 0.0
    rows[target, 0] = 1.0
    rows[:, 1] = torch.arange(n) / n            # tells the rows apart
    cache.pools[0].view(-1, rank)[pool_index(cache, 1, range(n))] = \
        rows.to(DEV, dtype)
    q = torch.zeros(H, 1 + count, rank)
    q[:, :, 0] = big
    out = latent_attention(q.to(DEV, dtype), None, cache.pools[0], b, rank,
                           1.0, window=window,
                           sink=None if sink is None else sink.to(DEV))
    return out[:, 1:].float().cpu(), rows


def _sees(pos, j, window):
    return j <= pos and (window <= 0 or pos - j < window)


def _check_crafted(out, rows, held, target, window, tol=2e-3):
    for i in range(out.shape[1]):
        pos = held + i
        hit = (out[:, i, 0] > 0.9).all().item()
        assert hit == _sees(pos, target, window), \
            "position %d, key %d, window %d" % (pos, target, window)
        if hit:
            assert (out[:, i] - rows[target]).abs().max() < tol


@pytest.mark.parametrize("target", [0, 1, 135, 136, 137, 150, 160, 161])
def test_decoded_token_sees_its_window_only(target):
    """One query at position 161 over 161 cached rows, window 25: the keys
    just inside (137) and just outside (136) the window, the first tokens,
    its neighbours and itself."""
    out, rows = _crafted_latent(161, 1, target, window=25)
    _check_crafted(out, rows, 161, target, 25)


@pytest.mark.parametrize("held,count,target", [
    (0, 40, 0), (0, 40, 13), (30, 20, 25), (30, 20, 29), (30, 20, 31),
    (61, 9, 56), (64, 2, 57), (7, 2, 0)])
def test_portion_queries_each_see_their_own_window(held, count, target):
    out, rows = _crafted_latent(held, count, target, window=9)
    _check_crafted(out, rows, held, target, 9)


@pytest.mark.parametrize("held,count,target", [
    (700, 1, 0), (700, 1, 3), (640, 3, 63), (640, 3, 64), (0, 300, 1)])
def test_a_far_key_among_hundreds_without_a_window(held, count, target):
    out, rows = _crafted_latent(held, count, target, window=0, block=64)
    _check_crafted(out, rows, held, target, 0)


def test_window_wider_than_the_sequence_and_window_of_one():
    out, rows = _crafted_latent(20, 5, 2, window=1000)
    _check_crafted(out, rows, 20, 2, 1000)
    out, rows = _crafted_latent(20, 5, 22, window=1)
    _check_crafted(out, rows, 20, 22, 1)


def test_sink_takes_its_share_of_the_weights_and_has_no_value():
    """The target scores ``big`` and everything else about 0: with a sink
    logit equal to that score the output is HALF the target's row, with a
    sink far below it the row itself; the sink is not scaled."""
    big = 30.0
    for s, share in ((big, 0.5), (big + math.log(3.0), 0.25), (-50.0, 1.0)):
        sink = torch.tensor([s, -50.0])          # head 1 has none to speak of
        out, rows = _crafted_latent(90, 3, 88, sink=sink, big=big)
        assert (out[0, :, 0] - share).abs().max() < 2e-3
        assert (out[1, :, 0] - 1.0).abs().max() < 2e-3
        assert (out[0] - share * rows[88]).abs().max() < 2e-3
    # scale applies to the scores but not to the sink
    from deepspeed_amd.ops.latent_attention import latent_attention
    cache, b = one_step_cache([4], {}, [0], [1])
    cache.pools[0].view(-1, 4)[pool_index(cache, 0, [0])] = \
        torch.tensor([[1.0, 0, 0, 0]]).to(DEV)
    q = torch.tensor([[[8.0, 0, 0, 0]]]).to(DEV)
    out = latent_attention(q, None, cache.pools[0], b, 4, 0.25,
                           sink=torch.tensor([2.0]).to(DEV))
    assert abs(out[0, 0, 0].item() - 0.5) < 1e-5   # exp(8/4) vs exp(2)


def _mixer_weights(cfg, i, seed):
    t = tensors(cfg, seed)
    return t, {k: v.double() for k, v in t.items()}


def _run_mixer(cfg, i, t, h, cuts, block=8):
    """Layer i's mixer of a one-layer-run model over one sequence in
    portions; returns its output rows."""
    model = build_model(strip(cfg), torch.float32, t).load_named_tensors(t) \
        .to(DEV).eval()
    cache = model.build_cache(2, 256, dtype=torch.float32, device=DEV,
                              block_size=block)
    cache.reset_slot(1)
    layer = model.layers[i]
    run = [r for r, (j, _) in enumerate(model.runs) if j == i][0]
    out, at = [], 0
    for c in cuts:
        cache.begin_ragged([1], [c])
        st = {k: cache.states[f"{k}{run}"] for k in ("conv", "rec")
              if f"{k}{run}" in cache.states}
        out.append(layer.mixer(h[at:at + c].to(DEV), cache,
                               model.stream_of.get(run), st).double().cpu())
        cache.end_step()
        at += c
    return torch.cat(out)


CUTS = [[19], [1] * 19, [2, 1, 9, 2, 5], [2] * 9 + [1]]


@pytest.mark.parametrize("cuts", CUTS)
def test_latent_attention_matches_oracle_over_cuts(cuts):
    cfg = config([(la(dims=2), None)])
    t, w = _mixer_weights(cfg, 0, 5)
    h = torch.randn(19, 24, generator=torch.Generator().manual_seed(1))
    want = O.latent_attention(h.double(), w, "l0.mix.",
                              cfg["layers"][0]["mixer"], 1e-5)
    close(_run_mixer(cfg, 0, t, h, cuts), want)


@pytest.mark.parametrize("cuts", CUTS)
def test_windowed_latent_attention_matches_oracle_over_cuts(cuts):
    cfg = config([(lw(win=5), None)])
    t, w = _mixer_weights(cfg, 0, 6)
    h = torch.randn(19, 24, generator=torch.Generator().manual_seed(2))
    want = O.latent_window_attention(h.double(), w, "l0.mix.",
                                     cfg["layers"][0]["mixer"], 1e-5)
    close(_run_mixer(cfg, 0, t, h, cuts), want)


@pytest.mark.parametrize("cuts", CUTS)
@pytest.mark.parametrize("kv,conv", [(2, 3), (4, 1), (1, 4)])
def test_channel_delta_matches_oracle_over_cuts(cuts, kv, conv):
    cfg = config([(cd(kv=kv, conv=conv), None)])
    t, w = _mixer_weights(cfg, 0, 7)
    h = torch.randn(19, 24, generator=torch.Generator().manual_seed(3))
    want = O.channel_delta(h.double(), w, "l0.mix.",
                           cfg["layers"][0]["mixer"], 1e-5)
    close(_run_mixer(cfg, 0, t, h, cuts), want)


def test_decay_per_channel_keeps_a_far_input_in_one_row_of_the_state():
    """Key channel 0 barely decays, the others vanish within a few tokens:
    after 300 tokens a query along channel 0 still reads the first token's
    value, a query along channel 1 reads nothing of it."""
    from deepspeed_amd.ops.linear_recurrence import linear_scan
    T, H, d, dv = 300, 2, 4, 3
    cache, _ = one_step_cache([], {"rec": ((H, d, dv), torch.float32)}, [0],
                              [1])
    decay = torch.full((T, H, d), 0.3)
    decay[:, :, 0] = 0.9999
    k = torch.zeros(T, H, d)
    k[0, :, 0] = k[0, :, 1] = 1.0                 # written once, at token 0
    v = torch.zeros(T, H, dv)
    v[0] = torch.tensor([[1.0, 2, 3], [4, 5, 6]])
    q = torch.zeros(T, H, d)
    q[:, 0, 0] = 1.0                              # head 0 asks channel 0
    q[:, 1, 1] = 1.0                              # head 1 asks channel 1
    beta = torch.ones(T, H)
    outs, at = [], 0
    for c in (1, 150, 2, 146, 1):                 # carried through the state
        b = cache.begin_ragged([0], [c])
        outs.append(linear_scan(*(x[at:at + c].contiguous().to(DEV)
                                  for x in (q, k, v, decay, beta)),
                                cache.states["rec"], b).cpu())
        cache.end_step()
        at += c
    o = torch.cat(outs)
    assert torch.allclose(o[-1, 0], v[0, 0] * 0.9999 ** 299, atol=1e-4)
    assert o[-1, 1].abs().max() < 1e-6
    assert torch.allclose(o[1, 1], v[0, 1] * 0.3, atol=1e-5)


def test_softplus_decay_and_sigmoid_gated_head_norm():
    from deepspeed_amd.ops.linear_recurrence import (head_norm_gate,
                                                     softplus_decay)
    g = torch.Generator().manual_seed(4)
    T, H, d, dv, eps = 6, 3, 5, 4, 1e-5
    z = 3 * torch.randn(T, H * d + 3, generator=g).to(DEV)
    bias, a_log = torch.randn(H * d, generator=g).to(DEV), \
        torch.randn(H, generator=g).to(DEV)
    got = softplus_decay(z[:, 3:], bias, a_log, H)
    want = torch.exp(-torch.exp(a_log.double().cpu())[None, :, None]
                     * O.softplus(z[:, 3:].double().cpu() + bias.double().cpu())
                     .view(T, H, d))
    close(got.double().cpu(), want, 1e-5)
    o = torch.randn(T, H, dv, generator=g).to(DEV)
    w = torch.randn(dv, generator=g).to(DEV)
    gz = torch.randn(T, H * dv + 2, generator=g).to(DEV)
    got = head_norm_gate(o, w, gz[:, 2:], eps, torch.float32, act="sigmoid")
    want = (O.rms(o.double().cpu(), eps) * w.double().cpu()).reshape(T, -1) \
        * O.sigmoid(gz[:, 2:].double().cpu())
    close(got.double().cpu(), want, 1e-5)


def _same_picks(idx, w, want):
    """The same experts per token, weights within float rounding."""
    for i, ww, p in zip(idx.cpu().tolist(), w.cpu().tolist(), want):
        got = dict(zip(i, ww))
        assert sorted(got) == sorted(e for e, _ in p)
        for e, x in p:
            assert abs(got[e] - x) < 1e-5


@pytest.mark.parametrize("n,ident,top,count,keep", [
    (6, 1, 2, 3, 2), (8, 2, 3, 2, 1), (5, 0, 1, 1, 1), (12, 3, 4, 4, 2),
    (6, 0, 6, 3, 3)])
def test_grouped_softmax_router_against_the_oracle(n, ident, top, count,
                                                   keep):
    """Negative choice scores: corrections well below zero, so a group that
    is left out must count as minus infinity, not as 0."""
    from deepspeed_amd.moe.routed import grouped_topk
    g = torch.Generator().manual_seed(n * 10 + top)
    T, W = 50, 8
    h = torch.randn(T, W, generator=g)
    r = {"experts": n - ident, "identity": ident, "top": top, "scale": 1.7,
         "groups": {"count": count, "keep": keep}}
    w = {"x.router": torch.randn(n, W, generator=g),
         "x.correction": torch.randn(n, generator=g) * 0.3 - 0.4}
    want = O.route(h.double(), w, "x.", r)
    logits = (h.double() @ w["x.router"].double().t()).float().to(DEV)
    idx, wt = grouped_topk(logits, w["x.correction"].to(DEV), top, count,
                           keep, score="softmax", group_score="max",
                           renorm=True, scale=1.7)
    _same_picks(idx, wt, want)


def _routed_against_oracle(T, experts, identity, top, count, keep):
    cfg = config([(lw(), moe(experts=experts, top=top, identity=identity,
                             count=count, keep=keep, limit=0.8))])
    t = tensors(cfg, 9)
    w = {k: v.double() for k, v in t.items()}
    model = build_model(strip(cfg), torch.float32, t).load_named_tensors(t) \
        .to(DEV).eval()
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(T))
    want = O.moe_ff(h.double(), w, "l0.mlp.", cfg["layers"][0]["mlp"])
    close(model.layers[0].mlp(h.to(DEV)).double().cpu(), want)


@pytest.mark.parametrize("T", [3, 70])     # both expert paths
def test_more_picks_than_experts_when_most_outputs_are_identity(T):
    """One expert and three identity outputs, three picks: the picks of a
    token outnumber the rows the experts produce for it."""
    _routed_against_oracle(T, experts=1, identity=3, top=3, count=2, keep=2)


@pytest.mark.gpu
@pytest.mark.parametrize("T", [3, 70])
def test_identity_picks_on_the_combine_kernel(T):
    _routed_against_oracle(T, experts=1, identity=3, top=3, count=2, keep=2)
    _routed_against_oracle(T, experts=4, identity=2, top=3, count=3, keep=2)


@pytest.mark.parametrize("T", [3, 70])     # both expert paths
def test_routed_experts_with_identity_outputs_match_oracle(T):
    cfg = config([(lw(), moe(experts=4, top=3, identity=2, count=3, keep=2,
                             limit=0.8))])
    t = tensors(cfg, 9)
    w = {k: v.double() for k, v in t.items()}
    model = build_model(strip(cfg), torch.float32, t).load_named_tensors(t) \
        .to(DEV).eval()
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(T))
    want = O.moe_ff(h.double(), w, "l0.mlp.", cfg["layers"][0]["mlp"])
    got = model.layers[0].mlp(h.to(DEV)).double().cpu()
    close(got, want)
    picks = O.route(h.double(), w, "l0.mlp.", cfg["layers"][0]["mlp"]["router"])
    assert any(e >= 4 for p in picks for e, _ in p), "no identity pick drawn"


# ----------------------------------------------- the model, step by step
@pytest.fixture(scope="module")
def base():
    return Served(BASE)


def test_first_tokens(base):
    for n in (1, 2, 3, 4):
        t = toks(n, seed=n)
        close(base.run(t, [n]), base.oracle(t))


def test_prefill_equals_token_by_token(base):
    t = toks(26, seed=2)
    want = base.oracle(t)
    close(base.run(t, [26]), want)
    close(base.run(t, [1] * 26), want)


@pytest.mark.parametrize("cuts", [[2] * 13, [15, 1, 1, 9], [3, 5, 2, 16],
                                  [16, 10], [7, 2, 2, 2, 13]])
def test_portions_cut_anywhere(base, cuts):
    t = toks(26, seed=3)
    close(base.run(t, cuts), base.oracle(t))


def test_layer_streams_match_oracle(base):
    t = toks(14, seed=4)
    want = []
    base.oracle(t, want)
    b = base.batcher
    r = b.open("streams")
    b.cache.begin_ragged([r.slot], [len(t)])
    taps = []
    base.model(torch.tensor(t, device=DEV), kv_cache=b.cache, taps=taps)
    b.cache.end_step()
    b.close(r)
    assert len(taps) == len(want) == 7          # layers 1 and 2 run twice
    for got, ref in zip(taps, want):
        close(got.cpu().double(), ref)


def test_every_pass_of_the_loop_has_its_own_cache_and_state(base):
    cache = base.batcher.cache
    # runs: 0 lw | 1 cd, 2 la | 3 cd, 4 la | 5 la | 6 cd
    assert len(cache.pools) == 4
    assert {"rec1", "conv1", "rec3", "conv3", "rec6", "conv6", "prev"} == \
        set(cache.states)
    assert len(base.model.layers) == 5          # weights are stored once
    assert [a for _, a in base.model.runs] == \
        [False, False, False, True, False, False, False]


def test_unequal_batch_equals_each_alone(base):
    seqs = [toks(n, seed=20 + n) for n in (1, 9, 17, 30)]
    b = base.batcher
    reqs = [b.open("u%d" % i) for i in range(4)]
    first = b.feed([(r, s[:max(1, len(s) // 2)]) for r, s in zip(reqs, seqs)]) \
        .double().cpu()
    rest = [(r, s[max(1, len(s) // 2):]) for r, s in zip(reqs, seqs)
            if len(s) > 1]
    second = b.feed(rest).double().cpu()
    for r in reqs:
        b.close(r)
    a1 = a2 = 0
    for s in seqs:
        n1 = max(1, len(s) // 2)
        got = first[a1:a1 + n1]
        a1 += n1
        if len(s) > 1:
            got = torch.cat([got, second[a2:a2 + len(s) - n1]])
            a2 += len(s) - n1
        close(got, base.oracle(s))


def test_a_request_left_out_of_steps_goes_on_later(base):
    a, c = toks(20, seed=31), toks(12, seed=32)
    b = base.batcher
    ra, rc = b.open("left"), b.open("busy")
    got = [b.feed([(ra, a[:6]), (rc, c[:3])]).cpu()[:6]]
    b.feed([(rc, c[3:8])])
    b.feed([(rc, c[8:])])
    got.append(b.feed([(ra, a[6:])]).cpu())
    b.close(ra)
    b.close(rc)
    close(torch.cat(got).double(), base.oracle(a))


def test_blocks_and_slots_are_used_again():
    """A pool of 4 blocks of 16 and 2 slots serves 6 requests in turn, each
    leaving rows, states, convolution tails and a last token behind."""
    s = Served(BASE, slots=2, max_tokens=64, block=16)
    for k in range(6):
        t = toks(20 + k, seed=40 + k)
        other = toks(9, seed=80 + k)
        b = s.batcher
        r1, r2 = b.open("a%d" % k), b.open("b%d" % k)
        got = b.feed([(r1, t[:11]), (r2, other)]).cpu()[:11]
        got = torch.cat([got, b.feed([(r1, t[11:])]).cpu()])
        b.close(r1)
        b.close(r2)
        close(got.double(), s.oracle(t))
    assert s.batcher.cache.blocks_free() == 4


def test_pool_exhaustion_is_an_error_not_a_wrap():
    s = Served(BASE, slots=2, max_tokens=32, block=16)
    r = s.batcher.open("big")
    with pytest.raises(RuntimeError):
        s.batcher.feed([(r, toks(33))])


def test_long_decode_past_windows_and_block_borders(base):
    t = toks(120, seed=9)
    close(base.run(t, [5] + [1] * 115), base.oracle(t), 5e-4)


VARIANTS = {
    # sizes that the base makes equal or 1 are unequal or larger here
    "no_loop_one_head_full_rotation": config(
        [(la(heads=1, dim=2, rot=8, vdim=3, rank=4, q_rank=3, dims=8,
             base=7.0), dense(7)),
         (lw(heads=1, dim=4, vdim=4, rank=4, win=1), None)], width=16,
        logit_scale=1.0),
    "loop_over_the_last_layers_three_times": config(
        [(cd(heads=3, kv=1, dim=4, vdim=7, conv=1, a_rank=1, g_rank=1),
          dense(9)),
         (lw(heads=5, dim=4, vdim=2, rank=3, win=300), moe(
             ff=5, experts=6, top=1, identity=0, count=1, keep=1, scale=1.0)),
         (la(heads=4, dim=6, rot=2, vdim=5, rank=16, q_rank=24, dims=2),
          moe(ff=7, experts=2, top=3, identity=4, count=2, keep=2,
              limit=0.3, scale=0.5))],
        width=20, vocab=29, loop=(1, 3, 3), eps=1e-3,
        bigram=(3, 1, 1)),
    "whole_model_looped_once_more": config(
        [(cd(heads=2, kv=2, dim=3, vdim=3, conv=5, a_rank=6, g_rank=2), None),
         (la(heads=2, dim=4, rot=4, vdim=4, rank=6, q_rank=2, dims=4), None)],
        width=12, vocab=53, loop=(0, 2, 2), logit_scale=3.0,
        bigram=(101, 1000, 999)),
}


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes_and_orders(name):
    cfg = VARIANTS[name]
    s = Served(cfg, seed=3)
    t = toks(23, vocab=cfg["vocab"], seed=4)
    want = s.oracle(t)
    close(s.run(t, [23]), want)
    close(s.run(t, [4, 1, 1, 11, 2, 4]), want)


def test_bfloat16_stays_near_the_oracle():
    s = Served(BASE, dtype=torch.bfloat16)
    t = toks(30, seed=6)
    want = s.oracle(t)
    close_rms(s.run(t, [30]), want, 0.03, flips=0.1)
    close_rms(s.run(t, [7, 1, 20, 1, 1]), want, 0.03, flips=0.1)


def test_states_stay_32_bit_in_16_bit_serving():
    s = Served(BASE, dtype=torch.bfloat16)
    st = s.batcher.cache.states
    assert st["rec1"].dtype == st["rec6"].dtype == torch.float32
    assert st["conv1"].dtype == torch.bfloat16
    assert st["prev"].dtype == torch.int64
    assert s.batcher.cache.pools[0].dtype == torch.bfloat16
    assert s.model.layers[1].mixer.w_a2.dtype == torch.float32
    assert s.model.layers[0].ls1.dtype == torch.float32


# ---------------------------------------------- mid size, default 64-token blocks
def _mid_config():
    return config(
        [(lw(heads=4, dim=24, vdim=16, rank=40, win=48, scale=0.2),
          dense(150)),
         (cd(heads=4, kv=2, dim=32, vdim=24, conv=4, a_rank=8, g_rank=8),
          moe(ff=40, experts=10, top=3, identity=2, count=4, keep=2)),
         (la(heads=6, dim=16, rot=16, vdim=24, rank=48, q_rank=56, dims=16,
             base=3000.0, scale=0.18),
          moe(ff=40, experts=7, top=2, identity=1, count=2, keep=1)),
         (lw(heads=2, dim=64, vdim=32, rank=24, win=70, scale=0.12), None)],
        width=96, vocab=131, eps=1e-6, loop=(0, 3, 2))


def _mixed_schedule(dtype):
    """Three requests of 150, 70 and 5 tokens share steps: portions that end
    inside, on and one past a block border beside single tokens; the short
    one ends early and its slot serves a fourth request."""
    s = Served(_mid_config(), seed=5, dtype=dtype, slots=3, max_tokens=64 * 6,
               block=64)
    seqs = {"a": toks(150, 131, 1), "b": toks(70, 131, 2),
            "c": toks(5, 131, 3), "d": toks(40, 131, 4)}
    plan = [{"a": 63, "b": 1, "c": 5}, {"a": 1, "b": 64, "d": 2},
            {"a": 1, "b": 1, "d": 30}, {"a": 64, "b": 1, "d": 1},
            {"a": 1, "b": 1, "d": 7}, {"a": 20, "b": 2}]
    b = s.batcher
    live, at, got = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in plan:
        entries = []
        for k, n in step.items():
            if k not in live:
                live[k] = b.open(k)
            entries.append((live[k], seqs[k][at[k]:at[k] + n]))
        out = b.feed(entries).double().cpu()
        o = 0
        for k, n in step.items():
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
            if at[k] == len(seqs[k]):
                b.close(live.pop(k))
    assert at == {k: len(v) for k, v in seqs.items()}
    return s, seqs, got


def test_mid_size_mixed_schedule_over_block_borders():
    s, seqs, got = _mixed_schedule(torch.float32)
    for k, t in seqs.items():
        close(torch.cat(got[k]), s.oracle(t), 5e-4)


# -------------------------------------------- the framework's entry points
def test_greedy_generation_through_the_scheduler(base):
    prompts = [toks(n, seed=60 + n) for n in (3, 12, 18)]
    b = base.batcher
    b.token_budget, b.prefill_chunk = 16, 7      # prompts enter in portions
    for i, p in enumerate(prompts):
        b.put(Request(uid=100 + i, prompt=torch.tensor(p), max_new_tokens=6))
    done = {r.uid: r.generated for r in b.run_to_completion()}
    b.token_budget, b.prefill_chunk = 2048, 0
    for i, p in enumerate(prompts):
        seq = list(p)
        for _ in range(6):
            seq.append(int(base.oracle(seq)[-1].argmax()))
        assert done[100 + i] == seq[len(p):]


def _save(folder, cfg, t):
    from safetensors.torch import save_file
    folder.mkdir(exist_ok=True)
    (folder / "config.json").write_text(json.dumps(strip(cfg)))
    save_file({k: v.bfloat16().contiguous() for k, v in t.items()},
              str(folder / "model.safetensors"))


def test_registry_loads_a_checkpoint_folder(tmp_path):
    cfg = VARIANTS["loop_over_the_last_layers_three_times"]
    t = {k: v.bfloat16().float() for k, v in tensors(cfg, seed=8).items()}
    _save(tmp_path, cfg, t)
    model = load_pretrained(str(tmp_path), dtype=torch.float32, device=DEV)
    assert model.architecture == "Numolorn"
    assert model.layers[0].mixer.a_rank == 1      # a size from the tensors
    b = ContinuousBatcher(model, max_slots=1, dtype=torch.float32,
                          device=torch.device(DEV), max_tokens=64)
    r = b.open("x")
    seq = toks(10, vocab=cfg["vocab"])
    got = b.feed([(r, seq)], rows=[9]).cpu().double()
    want = O.forward(seq, {k: v.double() for k, v in t.items()},
                     strip(cfg))[9:]
    close(got, want)
    # the parameters go back out under the checkpoint's names
    back = model.named_tensors()
    assert set(back) == set(t)
    for k, v in t.items():
        assert torch.equal(back[k].float().cpu(), v), k


def test_config_rejects_what_the_design_does_not_have():
    bad = strip(config([(la(), None)]))
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        build_model(bad)
    bad = strip(config([(la(), None)], loop=(0, 2, 2)))   # past the end
    with pytest.raises(ValueError):
        build_model(bad)
    bad = strip(config([(la(dims=3), None)]))             # odd rotation
    with pytest.raises(ValueError):
        build_model(bad)
    bad = strip(config([(cd(heads=3, kv=2), None)]))
    with pytest.raises(ValueError):
        build_model(bad)
    bad = strip(config([(lw(), {"kind": "glu", "ff": 8})]))
    with pytest.raises(ValueError):
        build_model(bad)
    bad = strip(config([(lw(), moe(experts=4, identity=1, count=2))]))
    with pytest.raises(ValueError):                        # 5 outputs, 2 groups
        build_model(bad)


def test_schedule_replay_runner(tmp_path):
    """bin/trace_run end to end: two requests, portions beside single tokens,
    a slot used again; logits files against the oracle."""
    import subprocess
    import sys
    import numpy as np
    cfg = BASE
    t = {k: v.bfloat16().float() for k, v in tensors(cfg, seed=11).items()}
    mdir, out = tmp_path / "m", tmp_path / "o"
    _save(mdir, cfg, t)
    a, b, c = toks(9, seed=1), toks(5, seed=2), toks(4, seed=3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]},
                                {"id": "b", "tokens": b[:2], "want": []}],
         "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [2]}],
         "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[6:7], "want": []}],
         "end": []},
        {"step": 3, "entries": [{"id": "a", "tokens": a[7:], "want": [0, 1]},
                                {"id": "c", "tokens": c, "want": [3]}],
         "end": ["a", "c"]},
    ]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run(
        [sys.executable, os.path.join(repo, "bin", "trace_run"), "--model",
         str(mdir), "--dtype", "float32", "--out", str(out), "--max-tokens",
         "128", "--slots", "2"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
        capture_output=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l.startswith("done")] == \
        ["done %d" % i for i in range(4)]
    w = {k: v.double() for k, v in t.items()}
    la_, lb, lc = (O.forward(s, w, strip(cfg)) for s in (a, b, c))
    want = {0: la_[[0, 5]], 1: lb[[4]], 3: torch.cat([la_[[7, 8]], lc[[3]]])}
    assert not (out / "2.f32").exists()
    for n, ref in want.items():
        got = np.fromfile(out / ("%d.f32" % n), dtype="<f4").reshape(
            ref.shape)
        close(torch.from_numpy(got).double(), ref)


def test_generate_command_line(tmp_path):
    """bin/ds_generate: registry -> init_inference -> generate, greedy."""
    import subprocess
    import sys
    cfg = VARIANTS["whole_model_looped_once_more"]
    t = {k: v.bfloat16().float() for k, v in tensors(cfg, seed=14).items()}
    _save(tmp_path, cfg, t)
    a, b = toks(6, 53, seed=70), toks(6, 53, seed=71)
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run(
        [sys.executable, os.path.join(repo, "bin", "ds_generate"),
         "--model-dir", str(tmp_path), "--dtype", "float32", "--max-new-tokens",
         "3", "--tokens", ",".join(map(str, a)), "--tokens",
         ",".join(map(str, b))], text=True, capture_output=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [json.loads(l) for l in p.stdout.split("\n")
             if l.startswith("{")]
    w = {k: v.double() for k, v in t.items()}
    for prompt, line in zip((a, b), lines):
        seq = list(prompt)
        for _ in range(3):
            seq.append(int(O.forward(seq, w, strip(cfg))[-1].argmax()))
        assert line["generated"] == seq[len(prompt):]


def test_http_server_generates_the_oracles_tokens():
    """The FastAPI front end over the same scheduler: concurrent requests,
    greedy tokens as the oracle's."""
    from concurrent.futures import ThreadPoolExecutor
    from fastapi.testclient import TestClient
    from deepspeed_amd.inference.server import InferenceServer, build_app
    s = Served(BASE, seed=21)
    prompts = [toks(n, seed=90 + n) for n in (5, 9, 3)]
    server = InferenceServer(s.model, max_slots=2).start()
    try:
        client = TestClient(build_app(server))

        def call(p):
            r = client.post("/generate", json={"token_ids": p,
                                               "max_new_tokens": 4})
            assert r.status_code == 200
            return r.json()["generated"]

        with ThreadPoolExecutor(3) as ex:
            got = list(ex.map(call, prompts))
    finally:
        server.stop()
    for p, g in zip(prompts, got):
        seq = list(p)
        for _ in range(4):
            seq.append(int(s.oracle(seq)[-1].argmax()))
        assert g == seq[len(p):]


# ------------------------------------------- HIP kernels against eager ops
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_match_eager_on_the_same_device(dtype, monkeypatch):
    from deepspeed_amd.ops import serving_kernels as sk
    t = toks(40, seed=12)
    s = Served(BASE, dtype=dtype)
    kern = s.run(t, [17, 1, 1, 21])
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    assert not sk.enabled()
    eager = s.run(t, [17, 1, 1, 21])
    if dtype == torch.float32:
        close(kern, eager, 1e-4)
    else:
        close_rms(kern, eager, 0.05, flips=0.1)


@pytest.mark.gpu
def test_kernel_libraries_are_loaded():
    from deepspeed_amd.ops import serving_kernels as sk
    Served(BASE).run(toks(5), [5])
    assert {"seq", "rows", "latent"} <= set(sk._libs)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mid_size_mixed_schedule_on_the_kernels(dtype):
    s, seqs, got = _mixed_schedule(dtype)
    for k, t in seqs.items():
        if dtype == torch.float32:
            close(torch.cat(got[k]), s.oracle(t), 5e-4)
        else:
            close_rms(torch.cat(got[k]), s.oracle(t), 0.03, flips=0.05)


@pytest.mark.gpu
@pytest.mark.parametrize("path", ["mfma", "exact"])
@pytest.mark.parametrize("held,count,target,window", [
    (161, 1, 137, 25), (161, 1, 136, 25), (30, 20, 29, 9), (64, 2, 57, 9),
    (700, 1, 3, 0), (0, 300, 1, 0), (500, 70, 470, 64), (500, 70, 436, 64),
    (500, 70, 437, 64)])
def test_tile_and_exact_attention_kernels_on_crafted_windows(
        path, held, count, target, window, monkeypatch):
    """Both kernels (bf16 tiles on the matrix cores, exact fp32) see the same
    keys at window edges; ``path`` is forced through the wrapper."""
    from deepspeed_amd.ops import serving_kernels as sk
    real = sk.latent_attention
    monkeypatch.setattr(sk, "latent_attention",
                        lambda *a, **k: real(*a, **{**k, "path": path}))
    dtype = torch.bfloat16 if path == "mfma" else torch.float32
    out, rows = _crafted_latent(held, count, target, window=window, rank=64,
                                block=64, dtype=dtype,
                                sink=torch.tensor([-40.0, -40.0]))
    _check_crafted(out, rows.to(dtype).float(), held, target, window,
                   tol=2e-2 if path == "mfma" else 2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,rank,rot,window,sink", [
    (4, 64, 0, 40, False), (5, 128, 32, 0, True), (8, 80, 0, 130, False),
    (3, 40, 8, 0, True), (16, 256, 64, 0, True), (2, 512, 0, 17, True)])
def test_latent_attention_kernels_against_eager(dtype, H, rank, rot, window,
                                                sink, monkeypatch):
    """Random rows, a batch of a long prompt portion, a decoded token over a
    long history and a fresh short prompt."""
    from deepspeed_amd.ops import serving_kernels as sk
    from deepspeed_amd.ops.latent_attention import latent_attention
    held, counts = [300, 777, 0], [150, 1, 9]
    cache, b = one_step_cache([rank + rot], {}, held, counts, block=64,
                              tokens=4096, dtype=dtype)
    g = torch.Generator().manual_seed(rank + rot)
    cache.pools[0].copy_(torch.randn(cache.pools[0].shape, generator=g)
                         .to(DEV, dtype))
    T = sum(counts)
    q = (torch.randn(H, T, rank, generator=g) * rank ** -0.5).to(DEV, dtype)
    qr = (torch.randn(T, H, rot, generator=g) * 0.3).to(DEV, dtype) \
        if rot else None
    sk_ = torch.randn(H, generator=g).to(DEV) if sink else None
    got = latent_attention(q, qr, cache.pools[0], b, rank, 0.7, window=window,
                           sink=sk_).float()
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    want = latent_attention(q, qr, cache.pools[0], b, rank, 0.7,
                            window=window, sink=sk_).float()
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    assert (got - want).abs().max().item() < tol * max(1.0, want.abs().max()
                                                       .item())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,taps", [
    (6, 3, 64, 48, 4), (4, 2, 128, 64, 4), (3, 1, 20, 12, 3),
    (8, 8, 32, 128, 2), (2, 2, 256, 16, 1)])
def test_channel_delta_kernels_against_eager(dtype, H, G, d, dv, taps,
                                             monkeypatch):
    from deepspeed_amd.ops.linear_recurrence import (delta_prep, linear_scan,
                                                     softplus_decay)
    C = 2 * G * d + H * dv
    wide = (C + H + 7) // 8 * 8
    held, counts = [37, 0, 5], [70, 1, 3]
    g = torch.Generator().manual_seed(H * d + taps)
    proj = torch.randn(sum(counts), wide, generator=g).to(DEV, dtype)
    conv_w = (0.5 * torch.randn(C, taps, generator=g)).to(DEV, dtype)
    z = torch.randn(sum(counts), H * d, generator=g).to(DEV)
    bias = torch.randn(H * d, generator=g).to(DEV)
    a_log = (torch.randn(H, generator=g) - 1).to(DEV)
    outs = []
    for eager in (False, True):
        if eager:
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        cache, b = one_step_cache(
            [], {"conv": ((max(taps - 1, 0), C), dtype),
                 "rec": ((H, d, dv), torch.float32)}, held, counts,
            tokens=1024, dtype=dtype)
        gs = torch.Generator().manual_seed(1)
        cache.states["conv"].copy_(torch.randn(cache.states["conv"].shape,
                                               generator=gs).to(DEV, dtype))
        cache.states["rec"].copy_(0.1 * torch.randn(
            cache.states["rec"].shape, generator=gs).to(DEV))
        for slot, n in enumerate(held):      # a new sequence starts from zero
            if n == 0:
                cache.states["conv"][slot].zero_()
                cache.states["rec"][slot].zero_()
        q, k, v, beta, none = delta_prep(proj, b, conv_w,
                                         cache.states["conv"], None, None, G,
                                         H, d, dv, beta_col=C, a_col=-1)
        assert none is None
        decay = softplus_decay(z, bias, a_log, H)
        o = linear_scan(q, k, v, decay, beta, cache.states["rec"], b)
        outs.append([x.float().clone() for x in
                     (q, k, v, beta, decay, o, cache.states["rec"],
                      cache.states["conv"])])
    for a, e in zip(*outs):
        if e.numel():                            # one tap carries no tail
            assert (a - e).abs().max().item() < \
                2e-4 * max(1.0, e.abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("C", [24, 192, 4096, 1000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scaled_add_kernel_against_eager(C, dtype, monkeypatch):
    from deepspeed_amd.ops.norms import scaled_add_
    g = torch.Generator().manual_seed(C)
    T = 7
    mk = lambda *s: torch.randn(*s, generator=g).to(DEV)
    x0, y1, y2, ex = mk(T, C), mk(T, C).to(dtype), mk(T, C).to(dtype), mk(T, C)
    s1, s2, w1, w2 = mk(C), mk(C), mk(C), mk(C)
    res = []
    for eager in (False, True):
        if eager:
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        for args in ((s1, y1, s2, y2, ex, w1, w2), (s1, y1, None, None, None,
                                                    w1, None),
                     (None, None, None, None, None, w1, w2),
                     (s1, y1, s2, y2, None, None, None)):
            x = x0.clone()
            h1, h2 = scaled_add_(x, *args, 1e-6, dtype)
            res.append([x] + [h.float() for h in (h1, h2) if h is not None])
    half = len(res) // 2
    for a, e in zip(res[:half], res[half:]):
        for u, v in zip(a, e):
            tol = 1e-5 if dtype == torch.float32 or u is a[0] else 1e-2
            assert (u - v).abs().max().item() < tol * max(1.0, v.abs().max()
                                                          .item())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("F", [96, 100, 4096])
def test_clamped_gate_kernel_against_eager(F, dtype, monkeypatch):
    """Eight columns per thread where the width allows, one otherwise."""
    from deepspeed_amd.ops.activations import clamped_swiglu
    gu = (2 * torch.randn(9, 2 * F, generator=torch.Generator()
                          .manual_seed(F))).to(DEV, dtype)
    got = clamped_swiglu(gu, 1.1).float()
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    want = clamped_swiglu(gu, 1.1).float()
    assert (got - want).abs().max().item() < \
        (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("E,top,count,keep,score,group", [
    (20, 4, 5, 2, "softmax", "max"), (10, 2, 5, 3, "softmax", "max"),
    (8, 2, 4, 2, "sigmoid", "top2"), (64, 8, 8, 4, "softmax", "top2"),
    (7, 7, 1, 1, "softmax", "max")])
def test_router_and_pair_hash_kernels_against_eager(E, top, count, keep,
                                                    score, group,
                                                    monkeypatch):
    from deepspeed_amd.moe.routed import grouped_topk
    from deepspeed_amd.ops.hashed_embedding import pair_hash_rows
    g = torch.Generator().manual_seed(E)
    z = (2 * torch.randn(300, E, generator=g)).to(DEV)
    corr = (0.3 * torch.randn(E, generator=g) - 0.2).to(DEV)
    cache = PagedStateCache([], {"prev": ((), torch.int64)}, 3, 4096,
                            block_size=64, device=DEV)
    ids = torch.randint(0, 50000, (300,), generator=g).to(DEV)
    res = []
    for eager in (False, True):
        if eager:
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        idx, w = grouped_topk(z, corr, top, count, keep, score=score,
                              group_score=group, renorm=score == "softmax",
                              scale=1.5)
        order = idx.argsort(-1)
        for s_ in range(3):
            cache.reset_slot(s_)
        cache.lens[1] = 70
        cache.states["prev"][1] = 123
        b = cache.begin_ragged([0, 1, 2], [200, 1, 99])
        rows = pair_hash_rows(ids, b, cache.states["prev"], 1009, 7, 65521)
        cache.end_step()
        res.append((idx.gather(-1, order), w.gather(-1, order), rows,
                    cache.states["prev"].clone()))
    assert torch.equal(res[0][0], res[1][0])
    assert (res[0][1] - res[1][1]).abs().max().item() < 1e-5
    assert torch.equal(res[0][2], res[1][2])
    assert torch.equal(res[0][3], res[1][3])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,v,gated", [(4, 32, True), (3, 6, True),
                                       (16, 128, False), (5, 20, False)])
def test_head_merge_kernel_against_eager(H, v, gated, dtype, monkeypatch):
    from deepspeed_amd.ops.latent_attention import gate_merge_heads
    g = torch.Generator().manual_seed(H * v)
    o = torch.randn(H, 37, v, generator=g).to(DEV, dtype)
    gate = torch.rand(37, H, generator=g).to(DEV) if gated else None
    got = gate_merge_heads(o, gate).float()
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    want = gate_merge_heads(o, gate).float()
    assert got.shape == (37, H * v)
    assert (got - want).abs().max().item() < \
        (1e-6 if dtype == torch.float32 else 2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,skip", [(6, 64, 0), (6, 64, 8), (3, 20, 0),
                                      (4, 128, 3)])
def test_decay_kernel_on_slices_against_eager(H, d, skip, dtype, monkeypatch):
    """Eight channels per thread where width, stride and address allow it,
    one otherwise (a slice that starts 3 columns in)."""
    from deepspeed_amd.ops.linear_recurrence import softplus_decay
    g = torch.Generator().manual_seed(H * d + skip)
    wide = (2 * torch.randn(29, H * d + 16, generator=g)).to(DEV, dtype)
    bias = torch.randn(H * d, generator=g).to(DEV)
    a_log = (torch.randn(H, generator=g) - 1).to(DEV)
    z = wide[:, skip:skip + H * d]
    got = softplus_decay(z, bias, a_log, H)
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    want = softplus_decay(z, bias, a_log, H)
    assert got.shape == (29, H, d) and got.dtype == torch.float32
    assert (got - want).abs().max().item() < 2e-6
