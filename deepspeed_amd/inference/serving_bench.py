"""Serving throughput of Fizesun beside Llama at equal width, depth and
feed-forward size, plus per-kernel distance from the roofline.

Random weights, synthetic tokens, bf16, one GPU. For every size:
* prefill: ``batch`` prompts of ``seq`` tokens in one ragged step (tokens/s);
* decode: ``batch`` requests holding ``seq`` tokens, one token each per step;
* kernels: each Fizesun kernel and the like kernel of the Llama path at the
  same shapes, timed alone, against max(bytes / HBM bandwidth, flops / MFMA
  peak). "distance" is measured time over that bound.
Run through ``python bench.py --serving fizesun``.

``--serving lolulorn`` does the same for Lolulorn (one block of gla /
attention / attention on borrowed rows / delta layers, dense and routed
feed-forwards) beside Llama, with Fizesun's throughput for the ragged path.

``--serving savovik`` runs Savovik (one block of mamba2 / capped windowed
attention / chunked attention beside a selective scan / mamba2 on the first
layer's weights) beside Lolulorn, its closest sibling on the ragged path, and
Llama; every Savovik kernel is timed next to the like Lolulorn kernel.

``--serving numolorn`` runs Numolorn (one block of windowed latent attention /
latent attention with sink and gate / two channel-decay delta layers, dense
and routed feed-forwards with identity outputs) beside Lolulorn (the closest
hybrid), Fizesun (the other latent-attention model) and Llama; every kernel on
its path is timed next to the like kernel of those paths.
"""

import json
import time

import torch

HBM_BW = 8.0e12          # bytes/s
MFMA_BF16 = 2.5e15       # flop/s dense

SIZES = {
    # width, layers, heads, ff, latent rank, rot, experts/top/expert ff
    "s": dict(width=1024, layers=4, heads=8, ff=4096, rank=128, rot=32,
              experts=8, top=2, eff=1024, batch=8, seq=1024),
    "m": dict(width=2048, layers=4, heads=16, ff=8192, rank=256, rot=64,
              experts=8, top=2, eff=2048, batch=8, seq=2048),
    "l": dict(width=4096, layers=2, heads=32, ff=14336, rank=512, rot=64,
              experts=8, top=2, eff=4096, batch=4, seq=4096),
}


def fizesun_config(z, vocab=32000):
    mix = {"heads": z["heads"], "dim": 128, "rot_dim": z["rot"], "vdim": 128,
           "kv_rank": z["rank"], "rot": {"base": 10000.0, "dims": z["rot"]},
           "scale": (128 + z["rot"]) ** -0.5}
    dense = {"kind": "dense", "ff": z["ff"]}
    moe = {"kind": "moe", "expert": {"ff": z["eff"], "limit": 7.0},
           "router": {"experts": z["experts"], "top": z["top"]},
           "shared": {"ff": z["eff"], "limit": 7.0}}
    layers = [{"type": "latent_attention", "mixer": mix,
               "mlp": dense if i % 2 == 0 else moe}
              for i in range(z["layers"])]
    return {"architecture": "Fizesun", "vocab": vocab, "width": z["width"],
            "norm": {"eps": 1e-6}, "canon": {"taps": 4}, "layers": layers}


def _timed(fn, warmup=2, iters=5):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters


def _fizesun_throughput(z, dev):
    from ..models.registry import build_model
    from .ragged import ContinuousBatcher
    model = build_model(fizesun_config(z), torch.bfloat16).init_random(0) \
        .to(dev).eval()
    B, S = z["batch"], z["seq"]
    b = ContinuousBatcher(model, max_slots=B, dtype=torch.bfloat16,
                          device=dev, max_tokens=B * (S + 64))
    g = torch.Generator().manual_seed(0)
    prompts = torch.randint(0, 32000, (B, S), generator=g).tolist()

    def prefill():
        reqs = [b.open(i) for i in range(B)]
        b.feed([(r, p) for r, p in zip(reqs, prompts)], rows=[0])
        return reqs

    def prefill_and_close():
        for r in prefill():
            b.close(r)

    t_pre = _timed(prefill_and_close, 1, 3)
    reqs = prefill()

    def decode():
        b.feed([(r, [7]) for r in reqs], rows=list(range(B)))

    t_dec = _timed(decode, 3, 20)
    for r in reqs:
        b.close(r)
    del model, b
    torch.cuda.empty_cache()
    return {"prefill_tok_s": B * S / t_pre, "decode_tok_s": B / t_dec,
            "decode_ms": 1e3 * t_dec}


def _llama_throughput(z, dev):
    from ..models import LlamaConfig, LlamaForCausalLM
    from .ragged import ContinuousBatcher, PagedKVCache
    B, S = z["batch"], z["seq"]
    cfg = LlamaConfig(vocab_size=32000, hidden_size=z["width"],
                      intermediate_size=z["ff"], num_layers=z["layers"],
                      num_heads=z["heads"], num_kv_heads=max(1, z["heads"] // 4),
                      max_seq_len=S + 64)
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).to(dev).eval()
    b = ContinuousBatcher(model, max_slots=B, max_seq=S + 64,
                          dtype=torch.bfloat16, device=dev,
                          cache_cls=PagedKVCache)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, 32000, (B, S), generator=g).to(dev)
    pos = torch.arange(S, dtype=torch.int32, device=dev).expand(B, S) \
        .contiguous()
    # prefill on the generate() path: contiguous cache, one batched forward
    from .kv_cache import StaticKVCache
    kv = StaticKVCache(cfg.num_layers, B, cfg.num_kv_heads, S + 64,
                       cfg.head_dim, dtype=torch.bfloat16, device=dev)

    @torch.no_grad()
    def prefill():
        kv.reset()
        model(ids, positions=pos, kv_cache=kv)

    t_pre = _timed(prefill, 1, 3)
    del kv
    last = torch.full((B, 1), 7, device=dev)

    def decode():
        for i in range(B):
            b.cache.lens[i] = S
        p = torch.full((B, 1), S, dtype=torch.int32, device=dev)
        b._forward(last, list(range(B)), 1, p)

    t_dec = _timed(decode, 3, 20)
    del model, b
    torch.cuda.empty_cache()
    return {"prefill_tok_s": B * S / t_pre, "decode_tok_s": B / t_dec,
            "decode_ms": 1e3 * t_dec}


@torch.no_grad()
def _kernel_rows(z, dev):
    """(name, like, seconds, bound seconds) per kernel at this size."""
    from ..ops import serving_kernels as sk
    from ..ops.attention import flash_attn_available, flash_attn_fwd
    from ..ops.norms import rms_norm
    from ..ops.paged_attention import paged_decode_attention
    from ..ops.swiglu import swiglu
    from .state_cache import PagedStateCache
    bf = torch.bfloat16
    B, S, W, H = z["batch"], z["seq"], z["width"], z["heads"]
    rank, rot, F = z["rank"], z["rot"], z["ff"]
    T = B * S
    out = []

    def row(name, like, fn, nbytes, flops=0.0):
        t = _timed(fn, 2, 5)
        bound = max(nbytes / HBM_BW, flops / MFMA_BF16)
        out.append({"kernel": name, "like": like, "us": 1e6 * t,
                    "bound_us": 1e6 * bound, "distance": t / bound})

    # ---- norm (+ conv) against RMSNorm
    cache = PagedStateCache([rank + rot], {"conv": (1, 3, W)}, B,
                            B * (S + 64), dtype=bf, device=dev)
    x32 = torch.randn(T, W, device=dev)
    x16 = x32.to(bf)
    gain = torch.ones(1, device=dev)
    cw = torch.randn(W, 4, device=dev).to(bf)
    wn = torch.ones(W, device=dev, dtype=bf)
    batch = cache.begin_ragged(list(range(B)), [S] * B)
    delta = torch.randn(T, W, device=dev).to(bf) * 0.01
    ssq = sk.residual_add_stats(x32, delta)
    row("norm_conv (fp32 stream in, bf16 out, 4 taps)", "rms_norm",
        lambda: sk.norm_conv_ragged(x32, gain, 1e-6, cw,
                                    cache.states["conv"][:, 0], batch, bf,
                                    ssq),
        T * W * 6)
    row("rms_norm (llama)", "", lambda: rms_norm(x16, wn, 1e-6), T * W * 4)
    row("residual_add_stats (fp32 stream += bf16, row sums)", "add",
        lambda: sk.residual_add_stats(x32, delta), T * W * 10)
    y16 = torch.empty_like(x16)
    row("add (llama residual, bf16)", "",
        lambda: torch.add(x16, delta, out=y16), T * W * 6)
    # ---- prefill attention
    q_lat = (torch.randn(H, T, rank, device=dev) * 0.1).to(bf)
    q_rot = (torch.randn(T, H, rot, device=dev) * 0.1).to(bf)
    cache.pools[0].normal_()
    fl = 2.0 * B * H * (S * S / 2) * (2 * rank + rot)
    row("latent_attention prefill (MFMA tiles)", "flash_attn_fwd",
        lambda: sk.latent_attention(q_lat, q_rot, cache.pools[0], batch, rank,
                                    0.07, path="mfma"),
        T * H * rank * 4 + T * (rank + rot) * 2, fl)
    q = torch.randn(B, S, H, 128, device=dev).to(bf)
    k = torch.randn(B, S, max(1, H // 4), 128, device=dev).to(bf)
    if flash_attn_available(q, k):
        row("flash_attn_fwd (llama)", "",
            lambda: flash_attn_fwd(q, k, k, causal=True),
            (2 * q.numel() + 2 * k.numel()) * 2,
            4.0 * B * H * (S * S / 2) * 128)
    cache.end_step()
    # ---- decode attention
    for i in range(B):
        cache.lens[i] = S
    batch = cache.begin_ragged(list(range(B)), [1] * B)
    qd_lat, qd_rot = q_lat[:, :B].contiguous(), q_rot[:B].contiguous()
    row("latent_attention decode (MFMA tiles, split keys)", "paged_decode",
        lambda: sk.latent_attention(qd_lat, qd_rot, cache.pools[0], batch,
                                    rank, 0.07),
        B * (S + 1) * (rank + rot) * 2)
    cache.end_step()
    hkv = max(1, H // 4)
    nb = B * ((S + 64) // 64)
    kp = torch.randn(nb, hkv, 64, 128, device=dev).to(bf)
    table = torch.arange(nb, dtype=torch.int32, device=dev).view(B, -1)
    lens = torch.full((B,), S + 1, dtype=torch.int32, device=dev)
    qd = torch.randn(B, H, 128, device=dev).to(bf)
    row("paged_decode (llama)", "",
        lambda: paged_decode_attention(qd, kp, kp, table, lens),
        B * (S + 1) * hkv * 128 * 2 * 2)
    # ---- the same at 64 requests, where the bytes of the cache matter
    NB = 64
    big = PagedStateCache([rank + rot], {}, NB, NB * (S + 64), dtype=bf,
                          device=dev)
    big.pools[0].normal_()
    for i in range(NB):
        big.lens[i] = S
    batch = big.begin_ragged(list(range(NB)), [1] * NB)
    qb_lat = (torch.randn(H, NB, rank, device=dev) * 0.1).to(bf)
    qb_rot = (torch.randn(NB, H, rot, device=dev) * 0.1).to(bf)
    row("latent_attention decode, 64 requests", "paged_decode",
        lambda: sk.latent_attention(qb_lat, qb_rot, big.pools[0], batch, rank,
                                    0.07),
        NB * (S + 1) * (rank + rot) * 2)
    big.end_step()
    del big
    nb = NB * ((S + 64) // 64)
    kp = torch.randn(nb, hkv, 64, 128, device=dev).to(bf)
    table = torch.arange(nb, dtype=torch.int32, device=dev).view(NB, -1)
    lens = torch.full((NB,), S + 1, dtype=torch.int32, device=dev)
    qd = torch.randn(NB, H, 128, device=dev).to(bf)
    row("paged_decode, 64 requests (llama)", "",
        lambda: paged_decode_attention(qd, kp, kp, table, lens),
        NB * (S + 1) * hkv * 128 * 2 * 2)
    del kp
    # ---- activations
    zf = torch.randn(T, F, device=dev).to(bf)
    pq = torch.zeros(2, device=dev)
    row("xielu", "swiglu", lambda: sk.xielu(zf, pq), T * F * 4)
    gu = torch.randn(T, 2 * F, device=dev).to(bf)
    row("clamped_swiglu", "swiglu", lambda: sk.clamped_swiglu(gu, 7.0),
        T * F * 6)
    up = torch.randn(T, F, device=dev).to(bf)
    row("swiglu (llama)", "", lambda: swiglu(zf, up), T * F * 6)
    return out


# ------------------------------------------------------------- Lolulorn
def lolulorn_config(z, vocab=32000):
    """One block [gla, attention, attention on the rows of the one before,
    delta] repeated to ``layers``; attention heads of 128 with 4 query heads
    per key/value head and a window of 1024 that keeps 4 first tokens;
    recurrent heads with keys of 128 and values of 256."""
    H = z["heads"]
    att = {"heads": H, "kv_heads": max(1, H // 4), "dim": 128, "vdim": 128,
           "scale": 128 ** -0.5, "mask": {"size": 1024, "keep_first": 4},
           "rot": {"base": 10000.0, "dims": 64, "scaling": {"factor": 2.0}}}
    gla = {"heads": max(1, H // 2), "dim": 128, "vdim": 256, "tau": 16.0,
           "rank": 16}
    delta = {"heads": max(1, H // 2), "kv_heads": max(1, H // 4), "dim": 128,
             "vdim": 256, "conv": 4}
    dense = {"kind": "dense", "ff": z["ff"]}
    moe = {"kind": "moe", "expert": {"ff": z["eff"]},
           "router": {"experts": z["experts"], "top": z["top"],
                      "groups": {"count": 4, "keep": 2}}}
    layers = []
    for i in range(z["layers"]):
        kind = i % 4
        if kind == 0:
            layers.append({"type": "gla", "mixer": gla, "mlp": dense})
        elif kind == 1:
            layers.append({"type": "attention", "mixer": att, "mlp": moe})
        elif kind == 2:
            layers.append({"type": "attention",
                           "mixer": {**att, "kv_from": i - 1}, "mlp": dense})
        else:
            layers.append({"type": "delta", "mixer": delta, "mlp": moe})
    return {"architecture": "Lolulorn", "vocab": vocab, "width": z["width"],
            "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
            "layers": layers}


def _ragged_throughput(cfg, z, dev):
    from ..models.registry import build_model
    from .ragged import ContinuousBatcher
    model = build_model(cfg, torch.bfloat16).init_random(0).to(dev).eval()
    B, S = z["batch"], z["seq"]
    b = ContinuousBatcher(model, max_slots=B, dtype=torch.bfloat16,
                          device=dev, max_tokens=B * (S + 64))
    g = torch.Generator().manual_seed(0)
    prompts = torch.randint(0, 32000, (B, S), generator=g).tolist()

    def prefill():
        reqs = [b.open(i) for i in range(B)]
        b.feed([(r, p) for r, p in zip(reqs, prompts)], rows=[0])
        return reqs

    def prefill_and_close():
        for r in prefill():
            b.close(r)

    t_pre = _timed(prefill_and_close, 1, 3)
    reqs = prefill()

    def decode():
        b.feed([(r, [7]) for r in reqs], rows=list(range(B)))

    t_dec = _timed(decode, 3, 20)
    for r in reqs:
        b.close(r)
    del model, b
    torch.cuda.empty_cache()
    return {"prefill_tok_s": B * S / t_pre, "decode_tok_s": B / t_dec,
            "decode_ms": 1e3 * t_dec}


@torch.no_grad()
def _lolulorn_kernel_rows(z, dev):
    """(name, like, seconds, bound seconds) per Lolulorn kernel at this size,
    each followed by the like kernel of the Llama path."""
    from ..ops import serving_kernels as sk
    from ..ops.attention import flash_attn_available, flash_attn_fwd
    from ..ops.norms import rms_norm
    from ..ops.paged_attention import paged_decode_attention
    from ..ops.rope import rope_tables
    from ..ops.swiglu import swiglu
    from .state_cache import PagedStateCache
    bf = torch.bfloat16
    B, S, W, H = z["batch"], z["seq"], z["width"], z["heads"]
    F = z["ff"]
    G, d, dv = max(1, H // 4), 128, 128
    win, keep = 1024, 4
    T = B * S
    out = []

    def row(name, like, fn, nbytes, flops=0.0, iters=5):
        t = _timed(fn, 2, iters)
        bound = max(nbytes / HBM_BW, flops / MFMA_BF16)
        out.append({"kernel": name, "like": like, "us": 1e6 * t,
                    "bound_us": 1e6 * bound, "distance": t / bound})

    # ---- post-norm + residual against RMSNorm and the bf16 residual add
    x32 = torch.randn(T, W, device=dev)
    x16 = x32.to(bf)
    y16 = (torch.randn(T, W, device=dev) * 0.01).to(bf)
    wn = torch.ones(W, device=dev)
    bn = torch.zeros(W, device=dev)
    row("layer_norm_add (fp32 stream += LN(bf16), bf16 copy)", "rms_norm+add",
        lambda: sk.layer_norm_add(x32, y16, wn, bn, 1e-6, bf), T * W * 12)
    wn16 = wn.to(bf)
    z16 = torch.empty_like(x16)
    row("rms_norm + add (llama)", "",
        lambda: torch.add(rms_norm(x16, wn16, 1e-6), y16, out=z16),
        T * W * 10)
    # ---- attention prologue and prefill
    cache = PagedStateCache([G * (d + dv)], {}, B, B * (S + 64), dtype=bf,
                            device=dev)
    batch = cache.begin_ragged(list(range(B)), [S] * B)
    cos, sin = rope_tables(64, cache.max_seq, 10000.0, device=dev, scaling=2.0)
    proj = torch.randn(T, (H + 2 * G) * d, device=dev).to(bf)
    qw, kw = torch.ones(H * d, device=dev), torch.ones(G * d, device=dev)
    row("attn_prep (q/k norm, rotary, cache write)", "rms_norm",
        lambda: sk.attn_prep(proj, batch, cache.pools[0], qw, kw, 1e-6, H, G,
                             d, dv, 64, cos, sin, True),
        T * (H + 2 * G) * d * 4)
    p16 = torch.randn(T, (H + 2 * G) * d, device=dev).to(bf)
    wp = torch.ones((H + 2 * G) * d, device=dev, dtype=bf)
    row("rms_norm over the same columns (llama)", "",
        lambda: rms_norm(p16, wp, 1e-6), T * (H + 2 * G) * d * 4)
    q = sk.attn_prep(proj, batch, cache.pools[0], qw, kw, 1e-6, H, G, d, dv,
                     64, cos, sin, True)
    seen = sum(min(i + 1, win) + min(keep, max(0, i + 1 - win))
               for i in range(S))
    row("window_attention prefill (window %d + %d kept)" % (win, keep),
        "flash_attn_fwd",
        lambda: sk.window_attention(q, cache.pools[0], batch, G, d, dv,
                                    d ** -0.5, win, keep),
        T * H * (d + dv) * 2 + T * G * (d + dv) * 2,
        2.0 * B * H * seen * (d + dv), iters=2)
    qf = torch.randn(B, S, H, 128, device=dev).to(bf)
    kf = torch.randn(B, S, G, 128, device=dev).to(bf)
    if flash_attn_available(qf, kf):
        row("flash_attn_fwd (llama, causal, no window)", "",
            lambda: flash_attn_fwd(qf, kf, kf, causal=True),
            (2 * qf.numel() + 2 * kf.numel()) * 2,
            4.0 * B * H * (S * S / 2) * 128)
    cache.end_step()
    # ---- decode attention at B and at 64 requests
    for NB in (B, 64):
        big = PagedStateCache([G * (d + dv)], {}, NB, NB * (S + 64), dtype=bf,
                              device=dev)
        big.pools[0].normal_()
        for i in range(NB):
            big.lens[i] = S
        bt = big.begin_ragged(list(range(NB)), [1] * NB)
        qd = (torch.randn(NB, H, d, device=dev) * 0.1).to(bf)
        vis = min(S + 1, win + keep)
        row("window_attention decode, %d requests" % NB, "paged_decode",
            lambda: sk.window_attention(qd, big.pools[0], bt, G, d, dv,
                                        d ** -0.5, win, keep),
            NB * vis * G * (d + dv) * 2)
        big.end_step()
        del big
        nb = NB * ((S + 64) // 64)
        kp = torch.randn(nb, G, 64, 128, device=dev).to(bf)
        table = torch.arange(nb, dtype=torch.int32, device=dev).view(NB, -1)
        lens = torch.full((NB,), S + 1, dtype=torch.int32, device=dev)
        qp = torch.randn(NB, H, 128, device=dev).to(bf)
        row("paged_decode, %d requests (llama, whole history)" % NB, "",
            lambda: paged_decode_attention(qp, kp, kp, table, lens),
            NB * (S + 1) * G * 128 * 2 * 2)
        del kp
    # ---- recurrences: no like kernel in the framework
    RH, RG, rd, rv = max(1, H // 2), max(1, H // 4), 128, 256
    for form in ("delta", "gla"):
        g_ = RG if form == "delta" else RH
        for NB, cnt in ((B, S), (B, 1), (64, 1)):
            rc = PagedStateCache([], {"rec": ((RH, rd, rv), torch.float32)},
                                 NB, NB * (S + 64), dtype=bf, device=dev)
            bt = rc.begin_ragged(list(range(NB)), [cnt] * NB)
            n = NB * cnt
            if form == "delta":
                qq = torch.randn(n, g_, rd, device=dev) * 0.1
                kk = torch.nn.functional.normalize(
                    torch.randn(n, g_, rd, device=dev), dim=-1)
                vv = torch.randn(n, RH, rv, device=dev)
                dec = torch.rand(n, RH, device=dev) * 0.1 + 0.9
                beta = torch.rand(n, RH, device=dev)
                io = n * (2 * g_ * rd + RH * rv) * 4
            else:
                qq = (torch.randn(n, g_, rd, device=dev) * 0.1).to(bf)
                kk = (torch.randn(n, g_, rd, device=dev) * 0.1).to(bf)
                vv = torch.randn(n, RH, rv, device=dev).to(bf)
                dec = torch.rand(n, RH, rd, device=dev) * 0.1 + 0.9
                beta = None
                io = n * (2 * g_ * rd + RH * rv) * 2 + n * RH * rd * 4
            st = rc.states["rec"]
            row("linear_scan %s, %d x %d tokens" % (form, NB, cnt), "",
                lambda: sk.linear_scan(qq, kk, vv, dec, beta, st, bt),
                io + n * RH * rv * 4 + 2 * NB * RH * rd * rv * 4,
                0.0)
            rc.end_step()
            del rc
    # ---- recurrence prologue / epilogue
    rc = PagedStateCache([], {"conv": (3, 2 * RG * rd + RH * rv)}, B,
                         B * (S + 64), dtype=bf, device=dev)
    bt = rc.begin_ragged(list(range(B)), [S] * B)
    C = 2 * RG * rd + RH * rv
    pj = torch.randn(T, C + RH * rv + 2 * RH, device=dev).to(bf)
    cw = torch.randn(C, 4, device=dev).to(bf)
    al, db = torch.zeros(RH, device=dev), torch.zeros(RH, device=dev)
    row("delta_prep (conv+silu, unit q/k, gates; fp32 out)", "norm_conv",
        lambda: sk.delta_prep(pj, bt, cw, rc.states["conv"], al, db, RG, RH,
                              rd, rv), T * C * 6)
    rc.end_step()
    o32 = torch.randn(T, RH, rv, device=dev)
    gate = torch.randn(T, RH * rv, device=dev).to(bf)
    nw = torch.ones(rv, device=dev)
    row("head_norm_gate (fp32 in, bf16 gate and out)", "rms_norm",
        lambda: sk.head_norm_gate(o32, nw, gate, 1e-6, bf), T * RH * rv * 8)
    # ---- activations
    gu = torch.randn(T, 2 * F, device=dev).to(bf)
    row("glu gelu_tanh", "swiglu", lambda: sk.glu(gu, 1), T * F * 6)
    row("glu silu", "swiglu", lambda: sk.glu(gu, 0), T * F * 6)
    zf = torch.randn(T, F, device=dev).to(bf)
    up = torch.randn(T, F, device=dev).to(bf)
    row("swiglu (llama)", "", lambda: swiglu(zf, up), T * F * 6)
    return out


def run_lolulorn(sizes=("s", "m", "l"), kernels=True):
    dev = torch.device("cuda", torch.cuda.current_device())
    report = {}
    for name in sizes:
        z = dict(SIZES[name])
        z["layers"] = 4 if name != "l" else 4
        rec = {"size": {k: z[k] for k in z},
               "lolulorn": _ragged_throughput(lolulorn_config(z), z, dev),
               "fizesun": _ragged_throughput(fizesun_config(z), z, dev),
               "llama": _llama_throughput(z, dev)}
        if kernels:
            rec["kernels"] = _lolulorn_kernel_rows(z, dev)
        report[name] = rec
        torch.cuda.empty_cache()
    return report



# -------------------------------------------------------------- Savovik
def savovik_config(z, vocab=32000):
    """One block [mamba2, attention, parallel, mamba2 on the first layer's
    weights] repeated to ``layers``: state-space heads of 64 with a state of
    128 (inner = 2 x width); attention heads of 128, 4 query heads per
    key/value head, window 1024, scores capped at 30; the parallel mixer's
    attention confined to chunks of 1024 beside a selective scan over
    ``width`` channels with 16 states each."""
    H, W = z["heads"], z["width"]
    att = {"heads": H, "kv_heads": max(1, H // 4), "dim": 128, "vdim": 128,
           "scale": 128 ** -0.5, "softcap": 30.0, "mask": {"size": 1024},
           "rot": {"base": 10000.0, "dims": 64, "scaling": {"factor": 2.0}}}
    left = {"heads": max(1, H // 2), "kv_heads": max(1, H // 8), "dim": 128,
            "vdim": 128, "scale": 128 ** -0.5, "mask": {"size": 1024},
            "rot": {"base": 500000.0, "dims": 64,
                    "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                                "original": 8192}}}
    right = {"inner": W, "state": 16, "dt_rank": max(1, W // 16), "conv": 4}
    m2 = {"heads": 2 * W // 64, "vdim": 64, "state": 128, "groups": 8,
          "norm_groups": 8, "conv": 4}
    dense = {"kind": "dense", "ff": z["ff"]}
    layers = []
    for i in range(z["layers"]):
        kind = i % 4
        if kind in (0, 3):
            spec = {"type": "mamba2", "mixer": m2, "mlp": dense}
            if kind == 3:
                spec["weights_of"] = i - 3
            layers.append(spec)
        elif kind == 1:
            layers.append({"type": "attention", "mixer": att, "mlp": dense})
        else:
            layers.append({"type": "parallel", "mlp": dense, "mixer": {
                "left": left, "right": right, "left_scale": 1.0,
                "right_scale": 1.0}})
    return {"architecture": "Savovik", "vocab": vocab, "width": W,
            "norm": {"eps": 1e-6}, "layers": layers}


@torch.no_grad()
def _savovik_kernel_rows(z, dev):
    """Every Savovik kernel at this size, each followed by the like kernel of
    the Lolulorn path ("like" names it; rows with an empty "like" are the
    siblings themselves)."""
    from ..ops import serving_kernels as sk
    from ..ops.rope import rope_tables
    from .state_cache import PagedStateCache
    bf = torch.bfloat16
    B, S, W, H = z["batch"], z["seq"], z["width"], z["heads"]
    F = z["ff"]
    G, d, dv = max(1, H // 4), 128, 128
    T = B * S
    out = []

    def row(name, like, fn, nbytes, flops=0.0, iters=5):
        t = _timed(fn, 2, iters)
        bound = max(nbytes / HBM_BW, flops / MFMA_BF16)
        out.append({"kernel": name, "like": like, "us": 1e6 * t,
                    "bound_us": 1e6 * bound, "distance": t / bound})

    # ---- gated residual (+ next norm) against the post-norm residual
    x32 = torch.randn(T, W, device=dev)
    side = torch.randn(T, 2 * W + 64, device=dev).to(bf)
    y1 = (torch.randn(T, W, device=dev) * 0.01).to(bf)
    y2 = (torch.randn(T, W, device=dev) * 0.01).to(bf)
    wn = torch.zeros(W, device=dev)
    row("gated_add (fp32 stream += 2 gated bf16 results, bf16 norm out)",
        "layer_norm_add",
        lambda: sk.gated_add(x32, side[:, :W], y1, side[:, W:2 * W], y2, wn,
                             1e-6, bf, True), T * W * 18)
    bn = torch.zeros(W, device=dev)
    row("layer_norm_add (lolulorn)", "",
        lambda: sk.layer_norm_add(x32, y1, wn + 1, bn, 1e-6, bf), T * W * 12)
    # ---- attention prologues
    cache = PagedStateCache([G * (d + dv)], {}, B, B * (S + 64), dtype=bf,
                            device=dev)
    batch = cache.begin_ragged(list(range(B)), [S] * B)
    cos, sin = rope_tables(64, cache.max_seq, 10000.0, device=dev, scaling=2.0)
    proj = torch.randn(T, (H + 2 * G) * d, device=dev).to(bf)
    hw = torch.ones(d, device=dev)
    nb = T * (H + 2 * G) * d * 4
    row("attn_prep: rotate-half, unit values, cache write", "attn_prep",
        lambda: sk.attn_prep(proj, batch, cache.pools[0], None, None, 1e-6, H,
                             G, d, dv, 64, cos, sin, True, None, "half",
                             1e-6), nb)
    row("attn_prep: per-head q/k norm, interleaved rotary, cache write",
        "attn_prep",
        lambda: sk.attn_prep(proj, batch, cache.pools[0], hw, hw, 1e-6, H, G,
                             d, dv, 64, cos, sin, True, "head", "interleaved",
                             None), nb)
    qw, kw = torch.ones(H * d, device=dev), torch.ones(G * d, device=dev)
    row("attn_prep (lolulorn: whole-projection norms)", "",
        lambda: sk.attn_prep(proj, batch, cache.pools[0], qw, kw, 1e-6, H, G,
                             d, dv, 64, cos, sin, True), nb)
    # ---- prefill attention
    q = sk.attn_prep(proj, batch, cache.pools[0], hw, hw, 1e-6, H, G, d, dv,
                     64, cos, sin, True, "head", "interleaved", None)
    win = 1024
    seen_w = sum(min(i + 1, win) for i in range(S))
    seen_c = sum(i % win + 1 for i in range(S))
    io = T * H * (d + dv) * 2 + T * G * (d + dv) * 2
    row("window_attention prefill (window %d, scores capped)" % win,
        "window_attention prefill",
        lambda: sk.window_attention(q, cache.pools[0], batch, G, d, dv,
                                    d ** -0.5, win, 0, None, 0, 30.0),
        io, 2.0 * B * H * seen_w * (d + dv), iters=2)
    row("window_attention prefill (chunks of %d)" % win,
        "window_attention prefill",
        lambda: sk.window_attention(q, cache.pools[0], batch, G, d, dv,
                                    d ** -0.5, 0, 0, None, win, 0.0),
        io, 2.0 * B * H * seen_c * (d + dv), iters=2)
    seen_l = sum(min(i + 1, win) + min(4, max(0, i + 1 - win))
                 for i in range(S))
    row("window_attention prefill (lolulorn: window %d + 4 kept)" % win, "",
        lambda: sk.window_attention(q, cache.pools[0], batch, G, d, dv,
                                    d ** -0.5, win, 4),
        io, 2.0 * B * H * seen_l * (d + dv), iters=2)
    cache.end_step()
    # ---- decode attention at B and at 64 requests
    for NB in (B, 64):
        big = PagedStateCache([G * (d + dv)], {}, NB, NB * (S + 64), dtype=bf,
                              device=dev)
        big.pools[0].normal_()
        for i in range(NB):
            big.lens[i] = S - 1          # the last token of a full chunk
        bt = big.begin_ragged(list(range(NB)), [1] * NB)
        qd = (torch.randn(NB, H, d, device=dev) * 0.1).to(bf)
        vis = min(S, win)
        nbytes = NB * vis * G * (d + dv) * 2
        row("window_attention decode (window, capped), %d requests" % NB,
            "window_attention decode",
            lambda: sk.window_attention(qd, big.pools[0], bt, G, d, dv,
                                        d ** -0.5, win, 0, None, 0, 30.0),
            nbytes)
        row("window_attention decode (chunk), %d requests" % NB,
            "window_attention decode",
            lambda: sk.window_attention(qd, big.pools[0], bt, G, d, dv,
                                        d ** -0.5, 0, 0, None, win, 0.0),
            nbytes)
        row("window_attention decode (lolulorn), %d requests" % NB, "",
            lambda: sk.window_attention(qd, big.pools[0], bt, G, d, dv,
                                        d ** -0.5, win, 4),
            NB * min(S, win + 4) * G * (d + dv) * 2)
        big.end_step()
        del big
    # ---- state-space prologue / epilogue against the delta rule's
    MH, P, N, MG = 2 * W // 64, 64, 128, 8
    inner, gn = MH * P, MG * N
    C = inner + 2 * gn
    rc = PagedStateCache([], {"conv": (3, C)}, B, B * (S + 64), dtype=bf,
                         device=dev)
    bt = rc.begin_ragged(list(range(B)), [S] * B)
    pj = torch.randn(T, inner + C + MH, device=dev).to(bf)
    cw = torch.randn(C, 4, device=dev).to(bf)
    cb = torch.zeros(C, device=dev)
    al, db = torch.zeros(MH, device=dev), torch.zeros(MH, device=dev)
    row("ssd_prep (conv+bias+silu, dt, decay; fp32 out)", "delta_prep",
        lambda: sk.ssd_prep(pj, bt, cw, cb, rc.states["conv"], al, db, MH, MG,
                            N, P), T * (C * 2 + inner * 8 + gn * 8))
    rc.end_step()
    RH, RG, rd, rv = max(1, H // 2), max(1, H // 4), 128, 256
    C2 = 2 * RG * rd + RH * rv
    rc = PagedStateCache([], {"conv": (3, C2)}, B, B * (S + 64), dtype=bf,
                         device=dev)
    bt = rc.begin_ragged(list(range(B)), [S] * B)
    pj2 = torch.randn(T, C2 + RH * rv + 2 * RH, device=dev).to(bf)
    cw2 = torch.randn(C2, 4, device=dev).to(bf)
    al2, db2 = torch.zeros(RH, device=dev), torch.zeros(RH, device=dev)
    row("delta_prep (lolulorn)", "",
        lambda: sk.delta_prep(pj2, bt, cw2, rc.states["conv"], al2, db2, RG,
                              RH, rd, rv), T * C2 * 6)
    rc.end_step()
    o32 = torch.randn(T, MH, P, device=dev)
    xx = torch.randn(T, MH, P, device=dev)
    gate = torch.randn(T, inner, device=dev).to(bf)
    skip = torch.ones(MH, device=dev)
    gw = torch.ones(inner, device=dev)
    row("gate_group_norm (fp32 o and x in, bf16 gate and out)",
        "head_norm_gate",
        lambda: sk.gate_group_norm(o32, xx, skip, gate, gw, 8, 1e-6, bf),
        T * inner * 12)
    o2 = torch.randn(T, RH, rv, device=dev)
    gate2 = torch.randn(T, RH * rv, device=dev).to(bf)
    nw = torch.ones(rv, device=dev)
    row("head_norm_gate (lolulorn)", "",
        lambda: sk.head_norm_gate(o2, nw, gate2, 1e-6, bf), T * RH * rv * 8)
    del o32, xx, gate, o2, gate2, pj, pj2
    # ---- the scans
    ch, SN = W, 16
    for NB, cnt in ((B, S), (B, 1), (64, 1)):
        n = NB * cnt
        rc = PagedStateCache([], {"rec": ((MH, N, P), torch.float32)}, NB,
                             NB * (S + 64), dtype=bf, device=dev)
        bt = rc.begin_ragged(list(range(NB)), [cnt] * NB)
        qq = torch.randn(n, MG, N, device=dev) * 0.1
        kk = torch.randn(n, MG, N, device=dev) * 0.1
        vv = torch.randn(n, MH, P, device=dev)
        dec = torch.rand(n, MH, device=dev) * 0.1 + 0.9
        st = rc.states["rec"]
        row("linear_scan mamba2 form, %d x %d tokens" % (NB, cnt),
            "linear_scan",
            lambda: sk.linear_scan(qq, kk, vv, dec, None, st, bt),
            n * (2 * MG * N + 2 * MH * P) * 4 + 2 * NB * MH * N * P * 4)
        rc.end_step()
        del rc, qq, kk, vv
        rc = PagedStateCache([], {"rec": ((ch, SN), torch.float32)}, NB,
                             NB * (S + 64), dtype=bf, device=dev)
        bt = rc.begin_ragged(list(range(NB)), [cnt] * NB)
        xs = torch.randn(n, ch, device=dev).to(bf)
        zs = torch.randn(n, ch, device=dev).to(bf)
        bc = (torch.randn(n, 2 * SN, device=dev) * 0.1).to(bf)
        dtp = torch.randn(n, ch, device=dev)
        a_log = torch.zeros(ch, SN, device=dev)
        zero = torch.zeros(ch, device=dev)
        so = torch.empty(n, ch, device=dev, dtype=bf)
        st2 = rc.states["rec"]
        row("selective_scan, %d x %d tokens" % (NB, cnt), "linear_scan",
            lambda: sk.selective_scan(xs, dtp, zero, a_log, bc[:, :SN],
                                      bc[:, SN:], zero, zs, st2, bt, 1.0, so),
            n * ch * 10 + n * 2 * SN * 2 + 2 * NB * ch * SN * 4)
        rc.end_step()
        del rc
        rc = PagedStateCache([], {"rec": ((RH, rd, rv), torch.float32)}, NB,
                             NB * (S + 64), dtype=bf, device=dev)
        bt = rc.begin_ragged(list(range(NB)), [cnt] * NB)
        qq = torch.randn(n, RG, rd, device=dev) * 0.1
        kk = torch.nn.functional.normalize(
            torch.randn(n, RG, rd, device=dev), dim=-1)
        vv = torch.randn(n, RH, rv, device=dev)
        dec = torch.rand(n, RH, device=dev) * 0.1 + 0.9
        beta = torch.rand(n, RH, device=dev)
        st3 = rc.states["rec"]
        row("linear_scan delta (lolulorn), %d x %d tokens" % (NB, cnt), "",
            lambda: sk.linear_scan(qq, kk, vv, dec, beta, st3, bt),
            n * (2 * RG * rd + 2 * RH * rv) * 4 + 2 * NB * RH * rd * rv * 4)
        rc.end_step()
        del rc, qq, kk, vv
    # ---- convolution of the selective scan's input, activations
    rc = PagedStateCache([], {"conv": (3, ch)}, B, B * (S + 64), dtype=bf,
                         device=dev)
    bt = rc.begin_ragged(list(range(B)), [S] * B)
    pin = torch.randn(T, 2 * ch + 64, device=dev).to(bf)
    cw3 = torch.randn(ch, 4, device=dev).to(bf)
    cb3 = torch.zeros(ch, device=dev)
    row("conv_silu (bias, bf16 in and out, 4 taps)", "delta_prep",
        lambda: sk.conv_silu_ragged(pin[:, 64:64 + ch], cw3,
                                    rc.states["conv"], bt, cb3, bf),
        T * ch * 4)
    rc.end_step()
    sd = torch.randn(T, 2 * W + F, device=dev).to(bf)
    row("act_rows gelu_erf (column slice)", "glu",
        lambda: sk.act_rows(sd[:, 2 * W:], 0), T * F * 4)
    gu = torch.randn(T, 2 * F, device=dev).to(bf)
    row("glu gelu_tanh (lolulorn)", "", lambda: sk.glu(gu, 1), T * F * 6)
    return out


def run_savovik(sizes=("s", "m", "l"), kernels=True):
    dev = torch.device("cuda", torch.cuda.current_device())
    report = {}
    for name in sizes:
        z = dict(SIZES[name])
        z["layers"] = 4
        rec = {"size": {k: z[k] for k in z},
               "savovik": _ragged_throughput(savovik_config(z), z, dev),
               "lolulorn": _ragged_throughput(lolulorn_config(z), z, dev),
               "llama": _llama_throughput(z, dev)}
        if kernels:
            rows = _savovik_kernel_rows(z, dev)
            rec["kernels"] = rows
            like = {}
            for r in rows:           # a sibling row follows the rows it is like
                if not r["like"]:
                    for q in rows:
                        if q["like"] and q["like"] in r["kernel"] \
                                and _same_case(q["kernel"], r["kernel"]):
                            like[q["kernel"]] = q["distance"] / r["distance"]
            rec["distance_over_sibling"] = like
        report[name] = rec
        torch.cuda.empty_cache()
    return report



# ------------------------------------------------------------- Numolorn
def numolorn_config(z, vocab=32000):
    """One block [windowed latent attention, latent attention with rotated
    part / sink / gate, channel-decay delta rule x 2] repeated to ``layers``;
    attention heads of 128 over a latent of ``rank``, window 1024; recurrent
    heads with keys of 128 and values of 256 as Lolulorn's; dense and routed
    feed-forwards of Lolulorn's sizes, two identity outputs beside the
    experts."""
    H, rank, rot = z["heads"], z["rank"], z["rot"]
    lw = {"heads": H, "dim": 128, "vdim": 128, "kv_rank": rank,
          "scale": 128 ** -0.5, "mask": {"size": 1024}}
    la = {"heads": H, "dim": 128, "rot_dim": rot, "vdim": 128,
          "kv_rank": rank, "q_rank": 3 * rank,
          "rot": {"base": 10000.0, "dims": rot},
          "scale": (128 + rot) ** -0.5}
    cd = {"heads": max(1, H // 2), "kv_heads": max(1, H // 4), "dim": 128,
          "vdim": 256, "conv": 4, "a_rank": 64, "g_rank": 64}
    dense = {"kind": "dense", "ff": z["ff"]}
    moe = {"kind": "moe", "expert": {"ff": z["eff"], "limit": 7.0},
           "router": {"experts": z["experts"], "top": z["top"], "identity": 2,
                      "scale": 1.5,
                      "groups": {"count": (z["experts"] + 2) // 2,
                                 "keep": 3}}}
    kinds = [("latent_attention_2", lw, dense), ("latent_attention", la, moe),
             ("channel_delta", cd, dense), ("channel_delta", cd, moe)]
    layers = [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1],
               "mlp": kinds[i % 4][2]} for i in range(z["layers"])]
    return {"architecture": "Numolorn", "vocab": vocab, "width": z["width"],
            "norm": {"eps": 1e-6}, "logit_scale": 1.0,
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 1009,
                                     "mul_cur": 7}},
            "layers": layers}


@torch.no_grad()
def _numolorn_kernel_rows(z, dev):
    """Every kernel on Numolorn's path at this size, each followed by the
    like kernel of the Lolulorn or Fizesun path at the same shapes ("like"
    names it; rows with an empty "like" are the siblings themselves)."""
    from ..ops import serving_kernels as sk
    from ..ops.rope import rope_tables
    from .state_cache import PagedStateCache
    bf = torch.bfloat16
    B, S, W, H = z["batch"], z["seq"], z["width"], z["heads"]
    rank, rot, F = z["rank"], z["rot"], z["ff"]
    d = 128
    T = B * S
    out = []

    def row(name, like, fn, nbytes, flops=0.0, iters=5):
        # the better of two runs: one slow allocation inside the timed calls
        # otherwise shows as a kernel several times off its bound
        t = min(_timed(fn, 2, iters), _timed(fn, 1, iters))
        bound = max(nbytes / HBM_BW, flops / MFMA_BF16)
        out.append({"kernel": name, "like": like, "us": 1e6 * t,
                    "bound_us": 1e6 * bound, "distance": t / bound})

    # ---- residual with learned factors (+ both norms of the next layer)
    x32 = torch.randn(T, W, device=dev)
    y1 = (torch.randn(T, W, device=dev) * 0.01).to(bf)
    y2 = (torch.randn(T, W, device=dev) * 0.01).to(bf)
    s1, s2 = torch.ones(W, device=dev), torch.ones(W, device=dev)
    wn, bn = torch.ones(W, device=dev), torch.zeros(W, device=dev)
    row("scaled_add (fp32 stream += 2 scaled bf16 results, 2 bf16 norms out)",
        "layer_norm_add",
        lambda: sk.scaled_add(x32, s1, y1, s2, y2, None, wn, wn, 1e-6, bf),
        T * W * 16)
    row("layer_norm_add (lolulorn)", "",
        lambda: sk.layer_norm_add(x32, y1, wn, bn, 1e-6, bf), T * W * 12)
    # ---- embedding: token row + hashed pair row
    emb = torch.randn(32000, W, device=dev).to(bf)
    pair = torch.randn(65522, W, device=dev).to(bf)
    ids = torch.randint(0, 32000, (T,), device=dev)
    pid = torch.randint(0, 65522, (T,), device=dev)
    row("embed_rows (two tables summed)", "embed_rows",
        lambda: sk.embed_rows(emb, ids, 1.0, torch.float32, pair, pid),
        T * W * 8)
    row("embed_rows (lolulorn: one table)", "",
        lambda: sk.embed_rows(emb, ids, 1.0, torch.float32), T * W * 6)
    del emb, pair
    # ---- latent prologue: operands from two products, rotate-half
    cache = PagedStateCache([rank + rot], {}, B, B * (S + 64), dtype=bf,
                            device=dev)
    batch = cache.begin_ragged(list(range(B)), [S] * B)
    cos, sin = rope_tables(rot, cache.max_seq, 10000.0, device=dev)
    nq = H * (d + rot)
    q = torch.randn(T, nq, device=dev).to(bf)
    side = torch.randn(T, rank + rot + H + 8, device=dev).to(bf)
    fused = torch.randn(T, nq + rank + rot + H, device=dev).to(bf)
    lw_ = torch.ones(rank, device=dev)
    nb = T * (nq + rank + rot) * 4
    row("latent_prep (q and latent from two products, rotate-half)",
        "latent_prep",
        lambda: sk.latent_prep(q, side[:, :rank + rot],
                               side[:, rank + rot:rank + rot + H], batch,
                               cache.pools[0], lw_, 1e-6, H, d, rot, rank,
                               rot, cos, sin, "half"), nb)
    row("latent_prep (fizesun: one fused row, neighbour pairs)", "",
        lambda: sk.latent_prep(fused[:, :nq], fused[:, nq:nq + rank + rot],
                               fused[:, nq + rank + rot:], batch,
                               cache.pools[0], lw_, 1e-6, H, d, rot, rank,
                               rot, cos, sin, "interleaved"), nb)
    cq = torch.randn(T, 3 * rank + 64, device=dev).to(bf)
    qn = torch.ones(3 * rank, device=dev)
    row("rms_norm_rows (query latent, a column slice)", "rms_norm_rows",
        lambda: sk.rms_norm_rows(cq[:, :3 * rank], qn, 1e-6, bf),
        T * 3 * rank * 4)
    cq2 = cq[:, :3 * rank].contiguous()
    row("rms_norm_rows (savovik: contiguous rows)", "",
        lambda: sk.rms_norm_rows(cq2, qn, 1e-6, bf), T * 3 * rank * 4)
    del q, side, fused, cq, cq2
    # ---- prefill attention over the latent rows
    q_lat = (torch.randn(H, T, rank, device=dev) * 0.1).to(bf)
    q_rot = (torch.randn(T, H, rot, device=dev) * 0.1).to(bf)
    cache.pools[0].normal_()
    sink = torch.zeros(H, device=dev)
    io = T * H * rank * 4 + T * (rank + rot) * 2
    fl = 2.0 * B * H * (S * S / 2) * (2 * rank + rot)
    row("latent_attention prefill (sink in the denominator)",
        "latent_attention prefill",
        lambda: sk.latent_attention(q_lat, q_rot, cache.pools[0], batch, rank,
                                    0.07, sink=sink), io, fl, iters=2)
    row("latent_attention prefill (fizesun)", "",
        lambda: sk.latent_attention(q_lat, q_rot, cache.pools[0], batch, rank,
                                    0.07), io, fl, iters=2)
    cache.end_step()
    win = 1024
    cw_ = PagedStateCache([rank], {}, B, B * (S + 64), dtype=bf, device=dev)
    bw = cw_.begin_ragged(list(range(B)), [S] * B)
    cw_.pools[0].normal_()
    seen = sum(min(i + 1, win) for i in range(S))
    row("latent_attention prefill (window %d, no rotated part)" % win,
        "window_attention prefill",
        lambda: sk.latent_attention(q_lat, None, cw_.pools[0], bw, rank, 0.07,
                                    window=win),
        T * H * rank * 4 + T * rank * 2, 2.0 * B * H * seen * 2 * rank,
        iters=2)
    cw_.end_step()
    del cw_, q_lat, q_rot
    G, dv = max(1, H // 4), 128
    ca = PagedStateCache([G * (d + dv)], {}, B, B * (S + 64), dtype=bf,
                         device=dev)
    ba = ca.begin_ragged(list(range(B)), [S] * B)
    ca.pools[0].normal_()
    qa = (torch.randn(T, H, d, device=dev) * 0.1).to(bf)
    seen_l = sum(min(i + 1, win) + min(4, max(0, i + 1 - win))
                 for i in range(S))
    row("window_attention prefill (lolulorn: window %d + 4 kept)" % win, "",
        lambda: sk.window_attention(qa, ca.pools[0], ba, G, d, dv, d ** -0.5,
                                    win, 4),
        T * H * (d + dv) * 2 + T * G * (d + dv) * 2,
        2.0 * B * H * seen_l * (d + dv), iters=2)
    ca.end_step()
    del ca, qa
    # ---- decode attention at B and at 64 requests
    for NB in (B, 64):
        big = PagedStateCache([rank + rot, rank], {}, NB, NB * (S + 64),
                              dtype=bf, device=dev)
        big.pools[0].normal_()
        big.pools[1].normal_()
        for i in range(NB):
            big.lens[i] = S
        bt = big.begin_ragged(list(range(NB)), [1] * NB)
        ql = (torch.randn(H, NB, rank, device=dev) * 0.1).to(bf)
        qr = (torch.randn(NB, H, rot, device=dev) * 0.1).to(bf)
        nbytes = NB * (S + 1) * (rank + rot) * 2
        row("latent_attention decode (sink), %d requests" % NB,
            "latent_attention decode",
            lambda: sk.latent_attention(ql, qr, big.pools[0], bt, rank, 0.07,
                                        sink=sink), nbytes)
        row("latent_attention decode (fizesun), %d requests" % NB, "",
            lambda: sk.latent_attention(ql, qr, big.pools[0], bt, rank, 0.07),
            nbytes)
        vis = min(S + 1, win)
        row("latent_attention decode (window %d), %d requests" % (win, NB),
            "window_attention decode",
            lambda: sk.latent_attention(ql, None, big.pools[1], bt, rank,
                                        0.07, window=win),
            NB * vis * rank * 2)
        big.end_step()
        del big
        big = PagedStateCache([G * (d + dv)], {}, NB, NB * (S + 64), dtype=bf,
                              device=dev)
        big.pools[0].normal_()
        for i in range(NB):
            big.lens[i] = S
        bt = big.begin_ragged(list(range(NB)), [1] * NB)
        qd = (torch.randn(NB, H, d, device=dev) * 0.1).to(bf)
        row("window_attention decode (lolulorn), %d requests" % NB, "",
            lambda: sk.window_attention(qd, big.pools[0], bt, G, d, dv,
                                        d ** -0.5, win, 4),
            NB * min(S + 1, win + 4) * G * (d + dv) * 2)
        big.end_step()
        del big
    # ---- the recurrence: a decay per key channel beside one per head
    RH, RG, rd, rv = max(1, H // 2), max(1, H // 4), 128, 256
    for NB, cnt in ((B, S), (B, 1), (64, 1)):
        rc = PagedStateCache([], {"rec": ((RH, rd, rv), torch.float32)}, NB,
                             NB * (S + 64), dtype=bf, device=dev)
        bt = rc.begin_ragged(list(range(NB)), [cnt] * NB)
        n = NB * cnt
        qq = torch.randn(n, RG, rd, device=dev) * 0.1
        kk = torch.nn.functional.normalize(torch.randn(n, RG, rd, device=dev),
                                           dim=-1)
        vv = torch.randn(n, RH, rv, device=dev)
        beta = torch.rand(n, RH, device=dev)
        dch = torch.rand(n, RH, rd, device=dev) * 0.1 + 0.9
        dhd = torch.rand(n, RH, device=dev) * 0.1 + 0.9
        st = rc.states["rec"]
        io = n * (2 * RG * rd + 2 * RH * rv) * 4 + 2 * NB * RH * rd * rv * 4
        row("linear_scan delta, decay per channel, %d x %d tokens"
            % (NB, cnt), "linear_scan delta",
            lambda: sk.linear_scan(qq, kk, vv, dch, beta, st, bt),
            io + n * RH * rd * 4)
        row("linear_scan delta (lolulorn: decay per head), %d x %d tokens"
            % (NB, cnt), "",
            lambda: sk.linear_scan(qq, kk, vv, dhd, beta, st, bt), io)
        rc.end_step()
        del rc
    # ---- recurrence prologue / epilogue
    C = 2 * RG * rd + RH * rv
    rc = PagedStateCache([], {"conv": (3, C)}, B, B * (S + 64), dtype=bf,
                         device=dev)
    bt = rc.begin_ragged(list(range(B)), [S] * B)
    pj = torch.randn(T, (C + RH + 128 + 7) // 8 * 8, device=dev).to(bf)
    pl = torch.randn(T, C + RH * rv + 2 * RH, device=dev).to(bf)
    cw = torch.randn(C, 4, device=dev).to(bf)
    al, db = torch.zeros(RH, device=dev), torch.zeros(RH, device=dev)
    row("delta_prep (conv+silu, unit q/k, beta; decay elsewhere)",
        "delta_prep",
        lambda: sk.delta_prep(pj, bt, cw, rc.states["conv"], None, None, RG,
                              RH, rd, rv, C, -1), T * C * 6)
    row("delta_prep (lolulorn: decay per head inside)", "",
        lambda: sk.delta_prep(pl, bt, cw, rc.states["conv"], al, db, RG, RH,
                              rd, rv), T * C * 6)
    rc.end_step()
    del pj, pl
    zz = torch.randn(T, RH * rd, device=dev)
    zb = torch.zeros(RH * rd, device=dev)
    row("softplus_decay (fp32 in and out, per key channel)", "sigmoid_pow",
        lambda: sk.softplus_decay(zz, zb, al, RH), T * RH * rd * 8)
    z16 = zz.to(bf)
    row("sigmoid_pow (lolulorn: bf16 in, fp32 out)", "",
        lambda: sk.sigmoid_pow(z16, zb, 1.0 / 16), T * RH * rd * 6)
    del zz, z16
    o32 = torch.randn(T, RH, rv, device=dev)
    gate = torch.randn(T, RH * rv, device=dev).to(bf)
    nw = torch.ones(rv, device=dev)
    row("head_norm_gate, sigmoid gate", "head_norm_gate",
        lambda: sk.head_norm_gate(o32, nw, gate, 1e-6, bf, "sigmoid"),
        T * RH * rv * 8)
    row("head_norm_gate (lolulorn: silu gate)", "",
        lambda: sk.head_norm_gate(o32, nw, gate, 1e-6, bf), T * RH * rv * 8)
    del o32, gate
    # ---- router and expert activation
    E = z["experts"] + 2
    lg = torch.randn(T, E, device=dev)
    corr = torch.zeros(E, device=dev)
    row("grouped_topk (softmax, best of group, renormalised)",
        "grouped_topk",
        lambda: sk.grouped_topk(lg, corr, z["top"], E // 2, 3, "softmax",
                                "max", True, 1.5), T * (E * 4 + z["top"] * 12))
    lg8 = torch.randn(T, z["experts"], device=dev)
    c8 = torch.zeros(z["experts"], device=dev)
    row("grouped_topk (lolulorn: sigmoid, two best of group)", "",
        lambda: sk.grouped_topk(lg8, c8, z["top"], 4, 2, "sigmoid", "top2",
                                False, 1.0),
        T * (z["experts"] * 4 + z["top"] * 12))
    gu = torch.randn(T, 2 * F, device=dev).to(bf)
    row("clamped_swiglu (experts)", "glu",
        lambda: sk.clamped_swiglu(gu, 7.0), T * F * 6)
    row("glu silu (lolulorn experts; numolorn dense)", "",
        lambda: sk.glu(gu, 0), T * F * 6)
    return out


def _sibling_ratios(rows):
    """distance of each row that names a like kernel over the distance of the
    sibling row that follows it (same case)."""
    like = {}
    for r in rows:
        if not r["like"]:
            for q in rows:
                if q["like"] and q["like"] in r["kernel"] \
                        and _same_case(q["kernel"], r["kernel"]):
                    like[q["kernel"]] = q["distance"] / r["distance"]
    return like


def run_numolorn(sizes=("s", "m", "l"), kernels=True):
    dev = torch.device("cuda", torch.cuda.current_device())
    report = {}
    for name in sizes:
        z = dict(SIZES[name])
        z["layers"] = 4
        rec = {"size": {k: z[k] for k in z},
               "numolorn": _ragged_throughput(numolorn_config(z), z, dev),
               "lolulorn": _ragged_throughput(lolulorn_config(z), z, dev),
               "fizesun": _ragged_throughput(fizesun_config(z), z, dev),
               "llama": _llama_throughput(z, dev)}
        if kernels:
            rows = _numolorn_kernel_rows(z, dev)
            rec["kernels"] = rows
            rec["distance_over_sibling"] = _sibling_ratios(rows)
        report[name] = rec
        torch.cuda.empty_cache()
    return report


def _same_case(a, b):
    """Rows of one case carry the same '<n> requests' / '<n> x <m> tokens'."""
    import re
    pat = r"(\d+ requests|\d+ x \d+ tokens)"
    return re.findall(pat, a) == re.findall(pat, b)

def run(sizes=("s", "m", "l"), kernels=True):
    dev = torch.device("cuda", torch.cuda.current_device())
    report = {}
    for name in sizes:
        z = SIZES[name]
        rec = {"size": {k: z[k] for k in z},
               "fizesun": _fizesun_throughput(z, dev),
               "llama": _llama_throughput(z, dev)}
        if kernels:
            rec["kernels"] = _kernel_rows(z, dev)
        report[name] = rec
        torch.cuda.empty_cache()
    return report


def main(sizes="s,m,l", out=None, model="fizesun"):
    names = tuple(sizes.split(","))
    if model == "numolorn":
        rep = run_numolorn(names)
        if out:
            with open(out, "w") as f:
                json.dump(rep, f, indent=1)
        best = rep[names[-1]]
        print(json.dumps({
            "metric": "numolorn_serving_tokens_per_s", "unit": "tokens/s",
            "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "value": best["numolorn"]["prefill_tok_s"],
            "higher_is_better": True,
            "sizes": {k: {"numolorn": v["numolorn"], "lolulorn": v["lolulorn"],
                          "fizesun": v["fizesun"], "llama": v["llama"],
                          "worst_distance_over_sibling": max(
                              v.get("distance_over_sibling", {}).values(),
                              default=None)}
                      for k, v in rep.items()}}))
        return rep
    if model == "savovik":
        rep = run_savovik(names)
        if out:
            with open(out, "w") as f:
                json.dump(rep, f, indent=1)
        best = rep[names[-1]]
        print(json.dumps({
            "metric": "savovik_serving_tokens_per_s", "unit": "tokens/s",
            "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "value": best["savovik"]["prefill_tok_s"],
            "higher_is_better": True,
            "sizes": {k: {"savovik": v["savovik"], "lolulorn": v["lolulorn"],
                          "llama": v["llama"],
                          "worst_distance_over_sibling": max(
                              v.get("distance_over_sibling", {}).values(),
                              default=None)}
                      for k, v in rep.items()}}))
        return rep
    rep = run(names) if model == "fizesun" else run_lolulorn(names)
    if out:
        with open(out, "w") as f:
            json.dump(rep, f, indent=1)
    best = rep[sizes.split(",")[-1]]
    extra = {} if model == "fizesun" else {"lolulorn": None}
    print(json.dumps({
        "metric": "%s_serving_tokens_per_s" % model, "unit": "tokens/s",
        "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
        "value": best[model]["prefill_tok_s"], "higher_is_better": True,
        "sizes": {k: {**{m: v[m] for m in extra}, "fizesun": v["fizesun"],
                      "llama": v["llama"],
                      "worst_kernel_distance": max(
                          (r["distance"] for r in v.get("kernels", [])
                           if r["like"]), default=None)}
                  for k, v in rep.items()}}))
    return rep
