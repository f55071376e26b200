"""Savovik through the serving path (registry -> ContinuousBatcher ->
PagedStateCache -> ops) against the plain oracle in savovik_oracle.py.

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

from tests import savovik_oracle as O
from deepspeed_amd.inference.ragged import ContinuousBatcher, Request
from deepspeed_amd.inference.state_cache import PagedStateCache
from deepspeed_amd.models import build_model, load_pretrained

DEV = "cuda" if torch.cuda.is_available() else "cpu"


# ------------------------------------------------------- configurations
def att(heads=4, kv=2, dim=8, vdim=6, win=9, dims=4, base=100.0, factor=1.5,
        scale=0.4, cap=5.0):
    return ("attention", {
        "heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
        "scale": scale, "softcap": cap, "mask": {"size": win},
        "rot": {"base": base, "dims": dims, "scaling": {"factor": factor}}})


def left(heads=2, kv=1, dim=6, vdim=10, chunk=7, dims=4, base=50.0,
         factor=3.0, low=1.0, high=3.0, original=24, scale=0.5):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
            "scale": scale, "mask": {"size": chunk},
            "rot": {"base": base, "dims": dims,
                    "scaling": {"factor": factor, "low": low, "high": high,
                                "original": original}}}


def right(inner=20, state=5, rank=3, conv=3):
    return {"inner": inner, "state": state, "dt_rank": rank, "conv": conv}


def par(l=None, r=None, ls=0.8, rs=1.3):
    return ("parallel", {"left": l or left(), "right": r or right(),
                         "left_scale": ls, "right_scale": rs})


def m2(heads=4, vdim=5, state=6, groups=2, parts=2, conv=4):
    return ("mamba2", {"heads": heads, "vdim": vdim, "state": state,
                       "groups": groups, "norm_groups": parts, "conv": conv})


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def config(layers, width=24, vocab=41, eps=1e-5):
    """layers: (mixer, mlp) pairs, or an int j for 'the weights of layer j'."""
    out = []
    for item in layers:
        if isinstance(item, int):
            out.append({**{k: v for k, v in out[item].items()
                           if k != "weights_of"}, "weights_of": item})
        else:
            (kind, mixer), mlp = item
            out.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Savovik", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "layers": out}


def tensors(cfg, seed=0):
    """Random tensors under the checkpoint's names, values that bfloat16
    holds exactly (so a saved folder reads back the same)."""
    g = torch.Generator().manual_seed(seed)
    W, t = cfg["width"], {}

    def rnd(*shape, s=1.0, shift=0.0):
        return ((torch.randn(*shape, generator=g) * s + shift)
                .bfloat16().float())

    def lin(o, i):
        return rnd(o, i, s=i ** -0.5)

    t["embed"] = rnd(cfg["vocab"], W)
    t["final.norm"] = rnd(W, s=0.2)
    t["head"] = lin(cfg["vocab"], W)
    for i, spec in enumerate(cfg["layers"]):
        if spec.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", spec["mixer"]
        t[p + "norm1"] = rnd(W, s=0.2)
        t[p + "rg1"], t[p + "rg1.b"] = lin(W, W), rnd(W, s=0.5)
        if spec["mlp"]:
            t[p + "rg2"], t[p + "rg2.b"] = lin(W, W), rnd(W, s=0.5)
            t[p + "mlp.up"] = lin(spec["mlp"]["ff"], W)
            t[p + "mlp.down"] = lin(W, spec["mlp"]["ff"])
        p += "mix."
        if spec["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[p + "q"], t[p + "k"] = lin(H * d, W) * 2, lin(G * d, W) * 2
            t[p + "v"], t[p + "o"] = lin(G * dv, W), lin(W, H * dv)
        elif spec["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, C = H * P, H * P + 2 * G * N
            t[p + "in"] = lin(inner + C + H, W)
            t[p + "conv"] = rnd(C, m["conv"], s=0.5)
            t[p + "conv.b"] = rnd(C, s=0.3)
            t[p + "dt_bias"] = rnd(H, s=0.5)
            t[p + "A_log"] = rnd(H, s=0.7, shift=-0.5)
            t[p + "D"] = rnd(H)
            t[p + "norm"] = rnd(inner, s=0.2, shift=1.0)
            t[p + "o"] = lin(W, inner)
        else:
            a, r = m["left"], m["right"]
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                t[p + "left." + n] = lin(rows, W) * (1 if n == "v" else 2)
                t[p + "left." + n + ".b"] = rnd(rows, s=0.3)
            t[p + "left.q.norm"] = rnd(d, s=0.2, shift=1.0)
            t[p + "left.k.norm"] = rnd(d, s=0.2, shift=1.0)
            t[p + "left.o"] = lin(W, H * dv)
            inner, N, R = r["inner"], r["state"], r["dt_rank"]
            t[p + "right.in"] = lin(2 * inner, W)
            t[p + "right.conv"] = rnd(inner, r["conv"], s=0.5)
            t[p + "right.conv.b"] = rnd(inner, s=0.3)
            t[p + "right.x"] = lin(R + 2 * N, inner)
            t[p + "right.dt"] = lin(inner, R)
            t[p + "right.dt.b"] = rnd(inner, s=0.5, shift=-1.0)
            t[p + "right.A_log"] = rnd(inner, N, s=0.7, shift=-0.5)
            t[p + "right.D"] = rnd(inner)
            t[p + "right.o"] = lin(W, inner)
    return t


BASE = config([(m2(), dense()), (att(), None), (par(), dense(28)), 0,
               (att(heads=2, kv=2, dim=4, vdim=4, win=5, dims=2), dense()),
               2])


class Served:
    """A configuration loaded into the framework plus its oracle weights."""

    def __init__(self, cfg, seed=0, dtype=torch.float32, slots=4,
                 max_tokens=512, block=16, t=None):
        self.cfg = cfg
        self.t = t or tensors(cfg, seed)
        self.w64 = {k: v.double() for k, v in self.t.items()}
        self.model = build_model(cfg, dtype).load_named_tensors(self.t) \
            .to(DEV).eval()
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


def close_rms(got, want, tol):
    """16-bit runs: root-mean-square error per position, against the spread."""
    err = ((got - want) ** 2).mean(-1).sqrt().max().item() / want.std().item()
    assert err < tol, "relative rms error %.3g" % err


def one_step_cache(row_dims, states, held, counts, block=8, tokens=512):
    """A cache whose slots already hold ``held`` tokens, with a step of
    ``counts`` new ones begun."""
    cache = PagedStateCache(row_dims, states, len(held), tokens,
                            block_size=block, device=DEV)
    for slot, n in enumerate(held):
        cache.reset_slot(slot)
        cache.lens[slot] = n
    return cache, cache.begin_ragged(list(range(len(held))), counts)


def pool_index(cache, slot, positions):
    bs, tab = cache.block_size, cache.block_table[slot]
    return torch.tensor([tab[p // bs] * bs + p % bs for p in positions]).to(DEV)


def in_steps(cache, slot, cuts, fn):
    """Run ``fn(batch, lo, hi)`` over one sequence cut into portions."""
    cache.reset_slot(slot)
    out, at = [], 0
    for c in cuts:
        b = cache.begin_ragged([slot], [c])
        out.append(fn(b, at, at + c))
        cache.end_step()
        at += c
    return torch.cat(out)


# ------------------------------------------------------ mechanisms alone
def test_norm_with_weights_around_zero_and_row_gather():
    from deepspeed_amd.ops.norms import rms_norm_rows
    torch.manual_seed(0)
    x, w = torch.randn(7, 24) * 3, torch.randn(24) * 0.3
    want = O.norm_one_plus(x.double(), w.double(), 1e-3)
    close(rms_norm_rows(x.to(DEV), w.to(DEV), 1e-3, torch.float32, None,
                        True).cpu().double(), want, 1e-5)
    idx = torch.tensor([5, 0, 5])
    close(rms_norm_rows(x.to(DEV), w.to(DEV), 1e-3, torch.float32,
                        idx.to(DEV), True).cpu().double(), want[idx], 1e-5)
    plain = O.rms(x.double(), 1e-3) * w.double()
    close(rms_norm_rows(x.to(DEV), w.to(DEV), 1e-3, torch.float32).cpu()
          .double(), plain, 1e-5)


@pytest.mark.parametrize("two", [False, True])
def test_gated_residual_and_the_norm_it_hands_on(two):
    from deepspeed_amd.ops.norms import gated_add_
    torch.manual_seed(1)
    T, C = 5, 24
    x, y1, y2 = torch.randn(T, C), torch.randn(T, C), torch.randn(T, C)
    side = torch.randn(T, 2 * C + 8)           # gates as column slices
    w = torch.randn(C) * 0.2
    want = x.double() + torch.sigmoid(side[:, :C].double()) * y1.double()
    if two:
        want = want + torch.sigmoid(side[:, C:2 * C].double()) * y2.double()
    xs, sd = x.clone().to(DEV), side.to(DEV)
    h = gated_add_(xs, sd[:, :C], y1.to(DEV), sd[:, C:2 * C] if two else None,
                   y2.to(DEV) if two else None, w.to(DEV), 1e-4,
                   torch.float32, True)
    close(xs.cpu().double(), want, 1e-5)
    close(h.cpu().double(), O.norm_one_plus(want, w.double(), 1e-4), 1e-5)
    xs = x.clone().to(DEV)
    assert gated_add_(xs, sd[:, :C], y1.to(DEV)) is None


def test_exact_gelu_on_a_column_slice():
    from deepspeed_amd.ops.activations import act_rows
    torch.manual_seed(2)
    z = torch.randn(6, 40) * 3
    got = act_rows(z.to(DEV)[:, 8:32], "gelu_erf").cpu().double()
    close(got, O.gelu_erf(z[:, 8:32].double()), 1e-5)
    tanh_form = act_rows(z.to(DEV), "gelu_tanh").cpu().double()
    assert (tanh_form - O.gelu_erf(z.double())).abs().max() > 1e-4


def test_three_band_frequencies():
    """One frequency in each band and the blend between them."""
    rot = {"base": 50.0, "dims": 12,
           "scaling": {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 24}}
    f = O.frequencies(rot)
    plain = torch.tensor([50.0 ** (-2.0 * i / 12) for i in range(6)],
                         dtype=torch.float64)
    waves = 2 * math.pi / plain
    kept, slowed = waves < 24 / 3.0, waves > 24 / 1.0
    assert kept.any() and slowed.any() and (~kept & ~slowed).any()
    assert torch.equal(f[kept], plain[kept])
    assert torch.allclose(f[slowed], plain[slowed] / 3.0)
    mid = ~kept & ~slowed
    assert ((f[mid] > plain[mid] / 3.0) & (f[mid] < plain[mid])).all()


@pytest.mark.parametrize("layout,scaling", [
    ("half", {"factor": 1.5}), ("half", None),
    ("interleaved", {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 24})])
def test_rotation_layouts_and_scalings(layout, scaling):
    """attn_prep's rotation at scattered positions against the oracle; the
    coordinates beyond rot.dims pass unchanged."""
    from deepspeed_amd.models.savovik import _rot_tables
    from deepspeed_amd.ops.window_attention import attn_prep
    torch.manual_seed(3)
    H, G, d, dv, dims = 2, 1, 10, 4, 6
    rot = {"base": 50.0, "dims": dims}
    if scaling:
        rot["scaling"] = scaling
    held = 37
    cache, b = one_step_cache([G * (d + dv)], {}, [held], [5], tokens=64)
    proj = torch.randn(5, H * d + G * d + G * dv)
    cos, sin = _rot_tables(rot, cache.max_seq, DEV)
    q = attn_prep(proj.to(DEV), b, cache.pools[0], None, None, 1e-6, H, G, d,
                  dv, dims, cos, sin, True, None, layout, None).cpu().double()
    want = O.rotate(proj[:, :H * d].double().reshape(5, H, d), rot, layout,
                    first_pos=held)
    close(q, want, 1e-5)
    assert torch.equal(q[..., dims:].float(),
                       proj[:, :H * d].reshape(5, H, d)[..., dims:])
    rows = cache.pools[0].view(-1, G * (d + dv))[pool_index(
        cache, 0, range(held, held + 5))].cpu().double()
    wk = O.rotate(proj[:, H * d:H * d + G * d].double().reshape(5, G, d), rot,
                  layout, first_pos=held)
    close(rows[:, :G * d], wk.reshape(5, -1), 1e-5)
    close(rows[:, G * d:], proj[:, H * d + G * d:].double(), 1e-6)


def test_per_head_norms_and_unit_values_in_the_cache():
    from deepspeed_amd.ops.window_attention import attn_prep
    torch.manual_seed(4)
    H, G, d, dv = 4, 2, 6, 5
    cache, b = one_step_cache([G * (d + dv)], {}, [3], [4], tokens=64)
    proj = torch.randn(4, H * d + G * d + G * dv) * 2
    wq, wk = torch.randn(d), torch.randn(d)
    q = attn_prep(proj.to(DEV), b, cache.pools[0], wq.to(DEV), wk.to(DEV),
                  1e-3, H, G, d, dv, 0, None, None, True, "head",
                  "interleaved", 1e-3).cpu().double()
    p = proj.double()
    close(q, O.rms(p[:, :H * d].reshape(4, H, d), 1e-3) * wq.double(), 1e-5)
    rows = cache.pools[0].view(-1, G * (d + dv))[pool_index(
        cache, 0, range(3, 7))].cpu().double()
    wantk = O.rms(p[:, H * d:H * d + G * d].reshape(4, G, d), 1e-3) * wk.double()
    close(rows[:, :G * d], wantk.reshape(4, -1), 1e-5)
    wantv = O.rms(p[:, H * d + G * d:].reshape(4, G, dv), 1e-3)
    close(rows[:, G * d:], wantv.reshape(4, -1), 1e-5)
    assert abs(float((rows[:, G * d:G * d + dv] ** 2).mean(-1)[0]) - 1) < 1e-2


def _crafted_attention(held, count, target, win=0, chunk=0, cap=0.0, G=2,
                       rep=2, dim=4, vdim=3, bs=8, score=40.0):
    """Rows 0..held+count-1 of one sequence; only row ``target`` has a key
    (``score`` against 0 for every head). Returns (out [count, H, vdim],
    values [L, G, vdim])."""
    from deepspeed_amd.ops.window_attention import window_attention
    g = torch.Generator().manual_seed(target + 7 * held)
    L = held + count
    cache, b = one_step_cache([G * (dim + vdim)], {}, [held], [count],
                              block=bs, tokens=L + bs)
    vals = torch.randn(L, G, vdim, generator=g)
    keys = torch.zeros(L, G, dim)
    if 0 <= target < L:
        keys[target, :, 0] = score
    rows = torch.cat([keys.reshape(L, -1), vals.reshape(L, -1)], 1)
    cache.pools[0].view(-1, rows.shape[1])[pool_index(cache, 0, range(L))] = \
        rows.to(DEV)
    q = torch.zeros(count, G * rep, dim)
    q[..., 0] = 1.0
    out = window_attention(q.to(DEV), cache.pools[0], b, G, dim, vdim, 1.0,
                           win, 0, None, chunk, cap).cpu() \
        .reshape(count, G * rep, vdim)
    cache.end_step()
    return out, vals


def _sees(pos, j, win, chunk):
    if j > pos:
        return False
    if win:
        return pos - j < win
    if chunk:
        return pos // chunk == j // chunk
    return True


def _check_crafted(out, vals, held, target, win=0, chunk=0, rep=2):
    for i in range(out.shape[0]):
        pos = held + i
        seen = [j for j in range(pos + 1) if _sees(pos, j, win, chunk)]
        for h in range(out.shape[1]):
            v = vals[:, h // rep].double()
            want = v[target] if target in seen else v[seen].mean(0)
            close(out[i, h].double(), want, 1e-4)


WIN, CHUNK = 20, 24


@pytest.mark.parametrize("target", [
    0, 7, 8, 150,                          # the start, a block border, far back
    299 - WIN, 299 - WIN + 1,              # just outside / inside for pos 299
    297, 299])
def test_decoded_token_sees_its_window_only(target):
    """A single query at position 299 over 300 rows in blocks of 8, and the
    same query one position before the target (which must not see it)."""
    out, vals = _crafted_attention(299, 1, target, win=WIN)
    _check_crafted(out, vals, 299, target, win=WIN)
    if target > 0:
        out, vals = _crafted_attention(target - 1, 1, target, win=WIN)
        _check_crafted(out, vals, target - 1, target, win=WIN)


@pytest.mark.parametrize("held,count,target", [
    (0, 40, 0), (0, 40, 19), (0, 40, 20), (30, 25, 11), (30, 25, 34),
    (30, 25, 35), (30, 25, 54), (61, 2, 42), (61, 2, 43), (61, 2, 62)])
def test_portion_queries_each_see_their_own_window(held, count, target):
    out, vals = _crafted_attention(held, count, target, win=WIN)
    _check_crafted(out, vals, held, target, win=WIN)


@pytest.mark.parametrize("pos,target", [
    (299, 0), (299, 150), (299, 287), (299, 288), (299, 299),  # chunk 12: 288..311
    (288, 287), (288, 288), (287, 264), (287, 263), (311, 288), (312, 311)])
def test_decoded_token_sees_its_chunk_only(pos, target):
    """Chunks of 24 counted from position 0 over blocks of 8: the last key of
    the chunk before is out, the chunk's first key is in."""
    out, vals = _crafted_attention(pos, 1, target, chunk=CHUNK)
    _check_crafted(out, vals, pos, target, chunk=CHUNK)


@pytest.mark.parametrize("held,count,target", [
    (0, 60, 0), (0, 60, 23), (0, 60, 24), (0, 60, 47), (0, 60, 48),
    (20, 10, 23), (20, 10, 24), (20, 10, 3), (47, 2, 47), (47, 2, 48),
    (47, 2, 24), (40, 80, 71), (40, 80, 72), (40, 80, 100)])
def test_portions_cross_chunk_edges_wherever_they_start(held, count, target):
    """A portion that begins mid-chunk and runs over one or more edges: every
    query's chunk is counted from the sequence's position 0."""
    out, vals = _crafted_attention(held, count, target, chunk=CHUNK)
    _check_crafted(out, vals, held, target, chunk=CHUNK)


def test_no_mask_and_masks_wider_than_the_sequence():
    for kw in ({}, {"win": 500}, {"chunk": 500}):
        out, vals = _crafted_attention(90, 3, 1, **kw)
        _check_crafted(out, vals, 90, 1, **kw)


def test_score_cap_levels_large_scores():
    """Two keys whose raw scores are 40 and 400: capped at 2 both weigh
    (almost) the same; uncapped the larger one takes everything."""
    from deepspeed_amd.ops.window_attention import window_attention
    G, dim, vdim, L = 1, 4, 3, 12
    cache, b = one_step_cache([G * (dim + vdim)], {}, [L - 1], [1],
                              tokens=64)
    g = torch.Generator().manual_seed(0)
    vals = torch.randn(L, vdim, generator=g)
    keys = torch.zeros(L, dim)
    keys[:, 0] = -400.0
    keys[3, 0], keys[8, 0] = 40.0, 400.0
    cache.pools[0].view(-1, dim + vdim)[pool_index(cache, 0, range(L))] = \
        torch.cat([keys, vals], 1).to(DEV)
    q = torch.zeros(1, 2, dim)
    q[..., 0] = 1.0
    capped = window_attention(q.to(DEV), cache.pools[0], b, G, dim, vdim, 1.0,
                              softcap=2.0).cpu().double().reshape(2, vdim)
    s = torch.full((L,), -400.0, dtype=torch.float64)
    s[3], s[8] = 40.0, 400.0
    w = torch.softmax(2.0 * torch.tanh(s / 2.0), 0)
    close(capped[0], w @ vals.double(), 1e-4)
    plain = window_attention(q.to(DEV), cache.pools[0], b, G, dim, vdim,
                             1.0).cpu().double().reshape(2, vdim)
    close(plain[1], vals[8].double(), 1e-4)


def test_attention_output_scaled_into_a_column_slice():
    from deepspeed_amd.ops.window_attention import window_attention
    out, vals = _crafted_attention(5, 3, 2)
    G, dim, vdim = 2, 4, 3
    cache, b = one_step_cache([G * (dim + vdim)], {}, [5], [3], tokens=64)
    keys = torch.zeros(8, G, dim)
    keys[2, :, 0] = 40.0
    g = torch.Generator().manual_seed(2 + 35)
    vals = torch.randn(8, G, vdim, generator=g)
    cache.pools[0].view(-1, G * (dim + vdim))[pool_index(
        cache, 0, range(8))] = torch.cat([keys.reshape(8, -1),
                                          vals.reshape(8, -1)], 1).to(DEV)
    q = torch.zeros(3, 4, dim)
    q[..., 0] = 1.0
    wide = torch.full((3, 4 * vdim + 5), 7.0, device=DEV)
    window_attention(q.to(DEV), cache.pools[0], b, G, dim, vdim, 1.0,
                     out_scale=0.5, out=wide[:, 5:])
    close(wide[:, 5:].cpu().double(), 0.5 * out.reshape(3, -1).double(), 1e-5)
    assert bool((wide[:, :5] == 7.0).all())


def _mixer_weights(kind, m, W, seed):
    cfg = config([((kind, m), None)], width=W)
    return cfg, {k: v.double() for k, v in tensors(cfg, seed).items()}


@pytest.mark.parametrize("cuts", [[19], [1] * 19, [2, 1, 9, 2, 5]])
def test_scalar_decay_mixer_matches_oracle_over_cuts(cuts):
    """The whole mamba2 mixer (prologue, scan, gated grouped norm) on one
    sequence, cut into portions."""
    from deepspeed_amd.models.savovik import Mamba2Mixer
    kind, m = m2(heads=6, vdim=3, state=5, groups=3, parts=2, conv=3)
    W = 16
    cfg, w = _mixer_weights(kind, m, W, 5)
    s = Served(cfg, seed=5)
    mixer = s.model.block(0).mixer
    assert isinstance(mixer, Mamba2Mixer)
    h = torch.randn(19, W, generator=torch.Generator().manual_seed(1))
    want = O.mamba2_mixer(h.double(), w, "l0.mix.", m, 1e-5)
    cache = s.batcher.cache
    st = {"conv": cache.states["conv0"], "rec": cache.states["rec0"]}
    got = in_steps(cache, 2, cuts, lambda b, lo, hi: mixer(
        h[lo:hi].to(DEV), cache, [], st).cpu().double())
    close(got, want, 1e-4)


@pytest.mark.parametrize("cuts", [[19], [1] * 19, [2, 1, 9, 2, 5]])
def test_parallel_mixer_matches_oracle_over_cuts(cuts):
    """Chunked attention beside the selective scan, one fused projection on
    either side, cut into portions that straddle chunk edges."""
    kind, m = par(left(heads=4, kv=2, dim=6, vdim=3, chunk=4),
                  right(inner=10, state=7, rank=2, conv=4), ls=0.7, rs=1.6)
    W = 16
    cfg, w = _mixer_weights(kind, m, W, 6)
    s = Served(cfg, seed=6)
    mixer = s.model.block(0).mixer
    h = torch.randn(19, W, generator=torch.Generator().manual_seed(2))
    want = O.parallel_mixer(h.double(), w, "l0.mix.", m, 1e-5)
    cache = s.batcher.cache
    st = {"conv": cache.states["conv0"], "rec": cache.states["rec0"]}
    got = in_steps(cache, 1, cuts, lambda b, lo, hi: mixer(
        h[lo:hi].to(DEV), cache, [0], st).cpu().double())
    close(got, want, 1e-4)


def test_selective_scan_keeps_a_far_input_by_its_decay():
    """One channel, one state: an input at token 3 and silence afterwards;
    the read-out 200 tokens later is the input times the product of the
    decays, whether the tokens come at once or one by one."""
    from deepspeed_amd.ops.selective_scan import selective_scan
    T, ch, N = 204, 3, 2
    x = torch.zeros(T, ch)
    x[3] = torch.tensor([1.0, 2.0, -1.0])
    dt_pre = torch.full((T, ch), -2.0)
    a_log = torch.tensor([[-3.0, -4.0]] * ch)
    B, C = torch.ones(T, N), torch.ones(T, N)
    z = torch.full((T, ch), 30.0)              # silu(30) = 30
    dt = math.log1p(math.exp(-2.0))
    for cuts in ([T], [4] + [1] * 200):
        cache = PagedStateCache([], {"rec": ((ch, N), torch.float32)}, 1, 256,
                                block_size=8, device=DEV)
        got = in_steps(cache, 0, cuts, lambda b, lo, hi: selective_scan(
            x[lo:hi].to(DEV), dt_pre[lo:hi].to(DEV), torch.zeros(ch).to(DEV),
            a_log.to(DEV), B[lo:hi].to(DEV), C[lo:hi].to(DEV),
            torch.zeros(ch).to(DEV), z[lo:hi].to(DEV), cache.states["rec"],
            b).cpu().double())
        want = sum(dt * math.exp(-math.exp(a) * dt * 200) for a in (-3.0, -4.0))
        close(got[203] / 30.0, torch.tensor([1.0, 2.0, -1.0]).double() * want,
              1e-4)
        assert float(got[2].abs().max()) == 0.0


def test_matrix_state_keeps_a_far_input_by_its_decay():
    """Scalar-decay recurrence through its prologue: one input at token 3,
    silence afterwards, constant B, C and step size; 200 tokens later the
    read-out is that input times the 200th power of the decay, whether the
    tokens come at once or one by one."""
    from deepspeed_amd.ops.linear_recurrence import linear_scan, ssd_prep
    T, H, P, G, N = 204, 1, 2, 1, 2
    proj = torch.zeros(T, 2 * H * P + 2 * G * N + H)
    proj[3, 2:4] = torch.tensor([1.0, -2.0])          # x before SiLU
    proj[:, 4:8] = 1.5                                 # B and C before SiLU
    proj[:, 8] = 0.3
    w, bias = torch.ones(H * P + 2 * G * N, 1), torch.zeros(H * P + 2 * G * N)
    a_log, dt_bias = torch.tensor([-2.0]), torch.tensor([-0.1])
    dt = math.log1p(math.exp(0.2))
    a = math.exp(-math.exp(-2.0) * dt)
    bc = float(O.silu(torch.tensor(1.5, dtype=torch.float64)))
    x3 = O.silu(torch.tensor([1.0, -2.0], dtype=torch.float64))
    want = N * bc * bc * dt * x3 * a ** 200
    for cuts in ([T], [4] + [1] * 200):
        cache = PagedStateCache([], {"conv": (0, H * P + 2 * G * N),
                                     "rec": ((H, N, P), torch.float32)}, 1,
                                256, block_size=8, device=DEV)

        def step(b, lo, hi):
            Cq, Bk, v, x, decay = ssd_prep(
                proj[lo:hi].to(DEV), b, w.to(DEV), bias.to(DEV),
                cache.states["conv"], a_log.to(DEV), dt_bias.to(DEV), H, G, N,
                P)
            return linear_scan(Cq, Bk, v, decay, None, cache.states["rec"],
                               b).cpu().double().reshape(hi - lo, P)
        got = in_steps(cache, 0, cuts, step)
        close(got[203], want, 1e-4)
        assert float(got[2].abs().max()) == 0.0


def test_short_convolution_with_bias_tail_carried_and_zero_at_the_start():
    from deepspeed_amd.ops.causal_conv import conv_silu_ragged
    torch.manual_seed(0)
    C, taps, S = 5, 4, 11
    x, w, bias = torch.randn(S, C + 3), torch.randn(C, taps), torch.randn(C)
    want = O.silu(O.causal_conv(x[:, 2:2 + C].double(), w.double(),
                                bias.double()))
    for cuts in ([11], [1] * 11, [2, 1, 6, 2]):
        cache = PagedStateCache([], {"conv": (taps - 1, C)}, 2, 64,
                                block_size=8, device=DEV)
        got = in_steps(cache, 1, cuts, lambda b, lo, hi: conv_silu_ragged(
            x[lo:hi].to(DEV)[:, 2:2 + C], w.to(DEV), cache.states["conv"], b,
            bias.to(DEV)).cpu().double())
        close(got, want, 1e-5)


def test_grouped_norm_after_the_gate():
    from deepspeed_amd.ops.linear_recurrence import gate_group_norm
    torch.manual_seed(7)
    T, H, P, parts = 4, 6, 5, 3
    o, x = torch.randn(T, H, P), torch.randn(T, H, P)
    skip, gate, w = torch.randn(H), torch.randn(T, H * P + 4), torch.randn(H * P)
    y = (o.double() + skip.double()[None, :, None] * x.double()) \
        .reshape(T, -1) * O.silu(gate[:, 4:].double())
    want = O.rms(y.reshape(T, parts, -1), 1e-3).reshape(T, -1) * w.double()
    got = gate_group_norm(o.to(DEV), x.to(DEV), skip.to(DEV),
                          gate.to(DEV)[:, 4:], w.to(DEV), parts, 1e-3,
                          torch.float32).cpu().double()
    close(got, want, 1e-5)


# ------------------------------------------------ whole model, schedules
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
    assert len(taps) == len(want) == len(BASE["layers"])
    for got, ref in zip(taps, want):
        close(got.cpu().double(), ref)


def test_a_layer_on_borrowed_weights_has_its_own_cache_and_state(base):
    cache = base.batcher.cache
    assert len(cache.pools) == 4               # layers 1, 2, 4 and 5
    assert {"rec0", "conv0", "rec2", "conv2", "rec3", "conv3", "rec5",
            "conv5"} == set(cache.states)
    assert len(base.model.blocks) == 4         # weights are stored once
    assert base.model.block(3) is base.model.block(0)


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
    leaving rows, states and convolution tails behind for the next."""
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


def test_long_decode_past_windows_chunks_and_block_borders(base):
    t = toks(120, seed=9)
    close(base.run(t, [5] + [1] * 115), base.oracle(t), 5e-4)


VARIANTS = {
    # sizes that the base makes equal or 1 are unequal or larger here
    "attention_only_mha_full_rotation": config(
        [(att(heads=3, kv=3, dim=6, vdim=9, win=4, dims=6, factor=1.0,
              cap=50.0), dense(7))], width=16),
    "mqa_window_of_one_then_wide": config(
        [(att(heads=5, kv=1, dim=4, vdim=4, win=1, dims=2), None),
         (att(heads=5, kv=1, dim=4, vdim=4, win=300, dims=4, cap=0.5), dense(11)),
         0, 1, 0], width=20, vocab=29),
    "single_group_single_part_single_tap": config(
        [(m2(heads=3, vdim=4, state=7, groups=1, parts=1, conv=1), None),
         (m2(heads=4, vdim=2, state=3, groups=4, parts=4, conv=2), dense(13))],
        width=12, eps=1e-3),
    "parallel_first_chunk_of_one": config(
        [(par(left(heads=3, kv=3, dim=4, vdim=4, chunk=1, dims=4),
              right(inner=6, state=1, rank=1, conv=1), ls=1.0, rs=1.0), None),
         (par(left(heads=6, kv=2, dim=8, vdim=2, chunk=50, dims=2, factor=8.0,
                   low=2.0, high=6.0, original=40),
              right(inner=9, state=17, rank=5, conv=5), ls=2.0, rs=0.25),
          dense(9)), 1], width=18, vocab=53),
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
    close_rms(s.run(t, [30]), want, 0.08)
    close_rms(s.run(t, [7, 1, 20, 1, 1]), want, 0.08)


def test_states_stay_32_bit_in_16_bit_serving():
    s = Served(BASE, dtype=torch.bfloat16)
    st = s.batcher.cache.states
    assert st["rec0"].dtype == st["rec2"].dtype == torch.float32
    assert st["conv0"].dtype == st["conv2"].dtype == torch.bfloat16
    assert s.batcher.cache.pools[0].dtype == torch.bfloat16
    assert s.model.block(2).mixer.w_dt.dtype == torch.float32


# ---------------------------------------------- mid size, default 64-token blocks
def _mid_config():
    return config(
        [(m2(heads=8, vdim=16, state=24, groups=2, parts=4, conv=4),
          dense(150)),
         (att(heads=8, kv=2, dim=24, vdim=20, win=40, dims=10, base=3000.0,
              factor=2.0, scale=0.2, cap=8.0), dense(100)),
         (par(left(heads=4, kv=2, dim=32, vdim=24, chunk=48, dims=16,
                   base=2000.0, factor=4.0, low=1.0, high=4.0, original=64,
                   scale=0.18),
              right(inner=136, state=12, rank=6, conv=4)), None),
         1, 0, 2], width=96, vocab=131, eps=1e-6)


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
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in t.items()},
              str(folder / "model.safetensors"))


def test_registry_loads_a_checkpoint_folder(tmp_path):
    cfg = VARIANTS["parallel_first_chunk_of_one"]
    t = tensors(cfg, seed=8)
    _save(tmp_path, cfg, t)
    model = load_pretrained(str(tmp_path), dtype=torch.float32, device=DEV)
    assert model.architecture == "Savovik"
    b = ContinuousBatcher(model, max_slots=1, dtype=torch.float32,
                          device=torch.device(DEV), max_tokens=64)
    r = b.open("x")
    seq = toks(10, vocab=cfg["vocab"])
    got = b.feed([(r, seq)], rows=[9]).cpu().double()
    want = O.forward(seq, {k: v.double() for k, v in t.items()}, cfg)[9:]
    close(got, want)


def test_config_rejects_what_the_design_does_not_have():
    bad = config([(att(), None)])
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        build_model(bad)
    bad = config([(att(), None), 0])
    bad["layers"][1]["weights_of"] = 1         # itself
    with pytest.raises(ValueError):
        build_model(bad)
    bad = config([(att(), None), 0])
    bad["layers"][1]["mixer"] = {**bad["layers"][1]["mixer"], "dim": 10}
    with pytest.raises(ValueError):
        build_model(bad)
    bad = config([(att(heads=3, kv=2), None)])
    with pytest.raises(ValueError):
        build_model(bad)
    bad = config([(att(), {"kind": "moe", "ff": 8})])
    with pytest.raises(ValueError):
        build_model(bad)


def test_schedule_replay_runner(tmp_path):
    """bin/trace_run end to end: two requests, portions beside single tokens,
    a slot used again; logits files against the oracle."""
    import subprocess
    import sys
    import numpy as np
    cfg = BASE
    t = tensors(cfg, seed=11)
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
    la, lb, lc = (O.forward(s, w, cfg) for s in (a, b, c))
    want = {0: la[[0, 5]], 1: lb[[4]], 3: torch.cat([la[[7, 8]], lc[[3]]])}
    assert not (out / "2.f32").exists()
    for n, ref in want.items():
        got = np.fromfile(out / ("%d.f32" % n), dtype="<f4").reshape(
            ref.shape)
        close(torch.from_numpy(got).double(), ref)


def test_generate_command_line(tmp_path):
    """bin/ds_generate: registry -> init_inference -> generate, greedy."""
    import subprocess
    import sys
    cfg = VARIANTS["mqa_window_of_one_then_wide"]
    t = tensors(cfg, seed=14)
    _save(tmp_path, cfg, t)
    a, b = toks(6, 29, seed=70), toks(6, 29, seed=71)
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
            seq.append(int(O.forward(seq, w, cfg)[-1].argmax()))
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
        close_rms(kern, eager, 0.05)


@pytest.mark.gpu
def test_sequence_library_is_loaded():
    from deepspeed_amd.ops import serving_kernels as sk
    Served(BASE).run(toks(5), [5])
    assert "seq" in sk._libs and "rows" in sk._libs


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mid_size_mixed_schedule_on_the_kernels(dtype):
    s, seqs, got = _mixed_schedule(dtype)
    for k, t in seqs.items():
        if dtype == torch.float32:
            close(torch.cat(got[k]), s.oracle(t), 5e-4)
        else:
            close_rms(torch.cat(got[k]), s.oracle(t), 0.08)


@pytest.mark.gpu
@pytest.mark.parametrize("ch,n", [(5, 1), (70, 16), (300, 24), (64, 40),
                                  (33, 100), (16, 200)])
def test_selective_scan_kernel_sizes_against_eager(ch, n, monkeypatch):
    from deepspeed_amd.ops import serving_kernels as sk
    from deepspeed_amd.ops.selective_scan import selective_scan
    g = torch.Generator().manual_seed(ch + n)
    counts = [9, 1, 30]
    T = sum(counts)

    def r(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(DEV)

    x, z, B, C = r(T, ch), r(T, ch), r(T, n), r(T, n)
    dt_pre, bias, a_log, skip = r(T, ch), r(ch), r(ch, n, s=0.5), r(ch)
    outs = []
    for eager in (False, True):
        if eager:
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        cache = PagedStateCache([], {"rec": ((ch, n), torch.float32)}, 3, 256,
                                block_size=8, device=DEV)
        cache.states["rec"].copy_(torch.randn(3, ch, n, generator=torch
                                              .Generator().manual_seed(1)))
        b = cache.begin_ragged([2, 0, 1], counts)
        outs.append((selective_scan(x, dt_pre, bias, a_log, B, C, skip, z,
                                    cache.states["rec"], b, out_scale=1.5)
                     .cpu().double(), cache.states["rec"].cpu().double()))
    assert not sk.enabled()
    close(outs[0][0], outs[1][0], 1e-4)
    close(outs[0][1], outs[1][1], 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,vdim,mask", [
    (20, 2, 24, 40, ("chunk", 33)), (3, 3, 128, 128, ("win", 70)),
    (8, 2, 48, 48, ("chunk", 64)), (4, 1, 256, 64, ("win", 200))])
def test_attention_kernel_masks_against_eager(dtype, heads, kv, dim, vdim,
                                              mask, monkeypatch):
    """Both attention kernels (exact for fp32, tiles for bf16) with the chunk
    mask, the window and the score cap, on portions and single tokens."""
    from deepspeed_amd.ops import window_attention as wa
    g = torch.Generator().manual_seed(heads + dim)
    held, counts = [130, 0, 257, 64], [70, 150, 1, 1]
    kw = {"chunk": mask[1]} if mask[0] == "chunk" else {"window": mask[1]}
    cache, b = one_step_cache([kv * (dim + vdim)], {}, held, counts, block=64,
                              tokens=64 * 16)
    cache.pools[0].copy_(torch.randn(cache.pools[0].shape, generator=g)
                         .to(dtype).to(DEV) if dtype == torch.float32 else
                         torch.randn(cache.pools[0].shape, generator=g))
    pool = cache.pools[0].to(dtype)
    q = torch.randn(sum(counts), heads, dim, generator=g).to(dtype).to(DEV)
    got = wa.window_attention(q, pool, b, kv, dim, vdim, dim ** -0.5,
                              softcap=3.0, out_scale=0.7, **kw).float().cpu()
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    want = wa.window_attention(q, pool, b, kv, dim, vdim, dim ** -0.5,
                               softcap=3.0, out_scale=0.7, **kw).float().cpu()
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert (got - want).abs().max().item() < tol * max(1.0, want.abs().max()
                                                       .item())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,vdim,dims,layout,norm,unit", [
    (8, 2, 128, 128, 64, "half", None, True),
    (8, 2, 128, 64, 64, "interleaved", "head", False),
    (4, 4, 256, 256, 128, "half", "head", True),
    (6, 3, 64, 32, 64, "interleaved", None, False),
    (3, 1, 40, 24, 16, "half", "head", True),
    (2, 2, 36, 20, 10, "half", "head", True),           # scalar form
    (5, 5, 48, 48, 24, "half", None, True)])            # half not a multiple of 8
def test_attention_prologue_sizes_against_eager(dtype, heads, kv, dim, vdim,
                                                dims, layout, norm, unit,
                                                monkeypatch):
    from deepspeed_amd.ops import window_attention as wa
    from deepspeed_amd.ops.rope import rope_tables
    g = torch.Generator().manual_seed(dim + vdim)
    held, counts = [5, 100], [40, 1]
    T = sum(counts)
    n = heads * dim + kv * (dim + vdim)
    wide = (torch.randn(T, n + 16, generator=g) * 2).to(dtype).to(DEV)
    proj = wide[:, 8:8 + n]                     # a column slice
    wq = (1 + 0.2 * torch.randn(dim, generator=g)).to(DEV)
    wk = (1 + 0.2 * torch.randn(dim, generator=g)).to(DEV)
    outs = []
    for eager in (False, True):
        if eager:
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        cache, b = one_step_cache([kv * (dim + vdim)], {}, held, counts,
                                  block=64, tokens=64 * 8)
        cache.pools[0] = cache.pools[0].to(dtype)
        cos, sin = rope_tables(dims, cache.max_seq, 1000.0, device=DEV,
                               scaling=2.0)
        q = wa.attn_prep(proj, b, cache.pools[0], wq, wk, 1e-5, heads, kv,
                         dim, vdim, dims, cos, sin, True, norm, layout,
                         1e-5 if unit else None)
        outs.append((q.float().cpu(), cache.pools[0].float().cpu()))
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for got, want in zip(*outs):
        assert (got - want).abs().max().item() < tol * max(
            1.0, want.abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim,state,groups,parts,taps", [
    (8, 64, 128, 2, 4, 4), (4, 16, 24, 4, 1, 3), (6, 8, 20, 3, 2, 2),
    (4, 32, 64, 1, 8, 5), (3, 5, 7, 3, 3, 4), (2, 64, 256, 2, 2, 1)])
def test_state_space_prologue_and_epilogue_against_eager(
        dtype, heads, vdim, state, groups, parts, taps, monkeypatch):
    from deepspeed_amd.ops.linear_recurrence import gate_group_norm, ssd_prep
    g = torch.Generator().manual_seed(heads * vdim + state)
    counts = [37, 1, 2]
    T = sum(counts)
    inner, C = heads * vdim, heads * vdim + 2 * groups * state
    proj = torch.randn(T, inner + C + heads, generator=g).to(dtype).to(DEV)
    w = (torch.randn(C, taps, generator=g) * 0.5).to(dtype).to(DEV)
    bias = torch.randn(C, generator=g).to(DEV)
    a_log, dt_bias = torch.randn(heads, generator=g).to(DEV), \
        torch.randn(heads, generator=g).to(DEV)
    skip, nw = torch.randn(heads, generator=g).to(DEV), \
        torch.randn(inner, generator=g).to(DEV)
    tail0 = torch.randn(3, max(taps - 1, 0), C, generator=g).to(dtype)
    held = (9, 70, 1)
    for slot, n in enumerate(held):             # nothing before position 0
        tail0[slot, :max(0, taps - 1 - n)] = 0
    outs = []
    for eager in (False, True):
        if eager:
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        cache = PagedStateCache([], {"conv": ((max(taps - 1, 0), C), dtype)},
                                3, 512, block_size=64, device=DEV)
        cache.states["conv"].copy_(tail0)
        for slot, n in enumerate(held):
            cache.lens[slot] = n
        b = cache.begin_ragged([0, 1, 2], counts)
        Cq, Bk, v, x, decay = ssd_prep(proj, b, w, bias, cache.states["conv"],
                                       a_log, dt_bias, heads, groups, state,
                                       vdim)
        y = gate_group_norm(v.contiguous(), x, skip, proj[:, :inner], nw,
                            parts, 1e-5, dtype)
        outs.append([t.float().cpu() for t in
                     (Cq, Bk, v, x, decay, y, cache.states["conv"])])
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for got, want in zip(*outs):
        if want.numel():                        # one tap keeps no tail
            assert (got - want).abs().max().item() < tol * max(
                1.0, want.abs().max().item())
