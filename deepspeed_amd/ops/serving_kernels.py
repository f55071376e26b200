"""ctypes front-end of the ragged-batch serving kernels
(csrc/serving/*.hip -> deepspeed_amd/ops/_serving*.so).

The libraries have a plain C ABI, so each builds with one hipcc call in a few
seconds and needs none of the torch headers; ``load()`` builds it on first use
when it is missing or older than its source. Wrappers take torch tensors,
check shapes and dtypes on the host (a kernel never sees operands it was not
written for) and launch on the current stream.

``enabled()`` is False on hosts without a GPU; the ops then use their torch
formulations. ``DS_AMD_SERVING_EAGER=1`` forces those on a GPU as well (a
debugging switch: kernels against eager on the same device).
"""

import ctypes
import os
import subprocess
import sys

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "csrc", "serving")
COMMON = os.path.join(_SRC, "serving_common.h")
# One library per family of mechanisms, each built from one source file: a
# model compiles and loads only the families its layers use.
#   rows   : norms, short convolutions, residual adds, activations, routers
#   latent : compressed-KV attention
#   seq    : windowed multi-head attention over paged K/V, linear recurrences
LIBRARIES = {
    "rows": (os.path.join(_SRC, "serving_kernels.hip"),
             os.path.join(_HERE, "_serving.so")),
    "latent": (os.path.join(_SRC, "latent_kernels.hip"),
               os.path.join(_HERE, "_serving_latent.so")),
    "seq": (os.path.join(_SRC, "sequence_kernels.hip"),
            os.path.join(_HERE, "_serving_seq.so")),
}
SOURCE, LIBRARY = LIBRARIES["rows"]
HIPCC_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-shared", "-fPIC"]

_libs = {}


def _compile(source, target):
    hipcc = os.environ.get("HIPCC") or (
        "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc")
        else "hipcc")
    tmp = "%s.%d.tmp" % (target, os.getpid())
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", tmp, source]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True)
    if r.returncode != 0:
        raise RuntimeError("building %s failed:\n%s"
                           % (os.path.basename(source), r.stdout))
    os.replace(tmp, target)
    return target


def _fresh(path, source):
    return os.path.exists(path) and \
        os.path.getmtime(path) >= max(os.path.getmtime(source),
                                      os.path.getmtime(COMMON))


def build(force=True, which=None):
    """Compile the libraries in-tree (cross-compiles without a GPU); ``which``
    names one family, default all. Returns the path of the (last) library.
    Where the tree cannot be written, a copy keyed by the sources' content
    goes to the temporary directory instead."""
    path = None
    for name in ([which] if which else list(LIBRARIES)):
        source, library = LIBRARIES[name]
        if not force and _fresh(library, source):
            path = library
        elif os.access(os.path.dirname(library), os.W_OK):
            path = _compile(source, library)
        else:
            import hashlib
            import tempfile
            tag = hashlib.sha1()
            for f in (COMMON, source):
                with open(f, "rb") as fh:
                    tag.update(fh.read())
            alt = os.path.join(tempfile.gettempdir(), "ds_amd_serving_%s_%s.so"
                               % (name, tag.hexdigest()[:16]))
            path = alt if os.path.exists(alt) else _compile(source, alt)
    return path


def load(which="rows"):
    lib = _libs.get(which)
    if lib is None:
        lib = _libs[which] = ctypes.CDLL(build(force=False, which=which))
        if which == "latent":
            lib.dsv_latent_attn_lds.restype = ctypes.c_int64
    return lib


def enabled() -> bool:
    return torch.cuda.is_available() and \
        os.environ.get("DS_AMD_SERVING_EAGER") != "1"


_DT = {torch.float32: 0, torch.bfloat16: 1}


def _dt(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"serving kernels take fp32 or bf16, not {t.dtype}")


def _p(t):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.is_cuda and t.is_contiguous(), "kernel operands are contiguous device tensors"
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _f(x):
    return ctypes.c_float(float(x))


def _i(x):
    return ctypes.c_int(int(x))


def _l(x):
    return ctypes.c_int64(int(x))


def _check(rc, name):
    if rc != 0:
        raise RuntimeError(f"{name}: launch refused or failed (code {rc})")


def _f32(t):
    return t if t.dtype == torch.float32 else t.float()


# ------------------------------------------------------------------ norm
def scalar_rms_norm(x, gain, eps, out_dtype, index=None):
    """out[r] = norm(x[index[r]] if index is given else x[r])."""
    assert x.dim() == 2
    rows = x.shape[0] if index is None else index.numel()
    out = torch.empty(rows, x.shape[1], dtype=out_dtype, device=x.device)
    if index is not None:
        index = index.to(torch.int64).contiguous()
    _check(load().dsv_scalar_rms_norm(
        _p(x), _i(_dt(x)), _p(index), _p(_f32(gain).reshape(1)), _p(out),
        _i(_DT[out_dtype]), _i(rows), _i(x.shape[1]), _f(eps), _stream()),
        "scalar_rms_norm")
    return out


def norm_conv_ragged(x, gain, eps, conv_w, state, batch, out_dtype,
                     sumsq=None):
    T, C = x.shape
    taps = conv_w.shape[1]
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert conv_w.dtype == out_dtype and state.dtype == out_dtype
    assert conv_w.shape[0] == C and conv_w.is_contiguous()
    assert state.shape[1:] == (taps - 1, C)
    assert state.stride(2) == 1 and (taps == 1 or state.stride(1) == C)
    assert T == batch.n_tokens
    assert sumsq is None or (sumsq.dtype == torch.float32
                             and sumsq.numel() == T)
    out = torch.empty(T, C, dtype=out_dtype, device=x.device)
    _check(load().dsv_norm_conv(
        _p(x), _p(_f32(gain).reshape(1)), _p(conv_w),
        ctypes.c_void_p(state.data_ptr()), _l(state.stride(0)),
        _p(batch.cu), _p(batch.seq_slot), _p(batch.seq_start),
        _p(batch.tok_seq), _p(batch.tok_pos), _p(out), _p(sumsq),
        _i(_DT[out_dtype]), _i(T), _i(batch.n_seqs), _i(C), _i(taps), _f(eps), _stream()),
        "norm_conv")
    return out


def residual_add_stats(x, delta):
    """x += delta in place; returns the per-row sums of squares of the new x."""
    T, C = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert delta.shape == x.shape
    delta = delta.contiguous()
    sumsq = torch.empty(T, dtype=torch.float32, device=x.device)
    _check(load().dsv_residual_add_stats(_p(x), _p(delta), _p(sumsq),
                                         _i(_dt(delta)), _i(T), _i(C),
                                         _stream()), "residual_add_stats")
    return sumsq


# ------------------------------------------------------ latent attention
def latent_prep(q, kv, gate_z, batch, pool, norm_w, eps, heads, dim, rot, rank,
                rot_dims, cos, sin, layout="interleaved"):
    """q [T, heads*(dim+rot)], kv [T, rank+rot], gate_z [T, heads] or None:
    column slices (rows contiguous) of one or of several projections."""
    T = q.shape[0]
    for t in (q, kv) + (() if gate_z is None else (gate_z,)):
        _rows_ok(t)
        assert t.dtype == pool.dtype and t.shape[0] == T
    assert q.shape[1] == heads * (dim + rot) and kv.shape[1] == rank + rot
    assert gate_z is None or gate_z.shape[1] == heads
    assert pool.shape[-1] == rank + rot and T == batch.n_tokens
    assert rot_dims % 2 == 0 and rot_dims <= rot
    assert layout in ("interleaved", "half")
    if rot_dims:
        assert cos.shape[1] == rot_dims // 2 and cos.shape[0] >= batch.max_ctx
        assert cos.dtype == torch.float32 and sin.shape == cos.shape
    dev, dt = q.device, q.dtype
    q_nope = torch.empty(heads, T, dim, dtype=dt, device=dev)
    q_rot = torch.empty(T, heads, rot, dtype=dt, device=dev) if rot else None
    gate = None if gate_z is None else \
        torch.empty(T, heads, dtype=torch.float32, device=dev)
    _check(load("latent").dsv_latent_prep(
        _vp(q), _i(q.stride(0)), _vp(kv), _i(kv.stride(0)),
        _p(None) if gate_z is None else _vp(gate_z),
        _i(0 if gate_z is None else gate_z.stride(0)), _p(_f32(norm_w)),
        _p(batch.tok_pos), _p(batch.tok_row), _p(cos if rot_dims else None),
        _p(sin if rot_dims else None), _p(pool), _p(q_nope), _p(q_rot),
        _p(gate), _i(_dt(q)), _i(T), _i(heads), _i(dim), _i(rot), _i(rank),
        _i(rot_dims), _f(eps), _i(1 if layout == "half" else 0), _stream()),
        "latent_prep")
    return q_nope, q_rot, gate


def _attn_plan(batch, dtype, rank, rot, reach=None):
    """Key-chunk length that fits LDS, and the number of key splits: few
    tokens over a long history are split so the launch still fills the chip.
    ``reach``: the most keys a token sees (a window bounds it)."""
    reach = batch.max_ctx if reach is None else reach
    lib = load("latent")
    dt = _DT[dtype]
    kc = 64
    while kc > 4 and lib.dsv_latent_attn_lds(dt, rank, rot, kc) > 60 * 1024:
        kc //= 2
    nsplit = 1
    if batch.n_tokens <= 128:
        nsplit = max(1, min(32, reach // (4 * kc),
                            1024 // max(1, batch.n_tokens)))
    return kc, nsplit


def _tile_work(batch, heads, tile_rows, device):
    """[(sequence, first row)] over every sequence's count*heads rows, late
    (long-history) tiles first so the heavy workgroups start early."""
    key = ("latent_tiles", heads, tile_rows)
    if key not in batch.extra:
        import numpy as np
        work = []
        for i, (st, c) in enumerate(zip(batch.starts, batch.counts)):
            for m0 in range(0, c * heads, tile_rows):
                work.append((st + (m0 + tile_rows) // heads, i, m0))
        work.sort(reverse=True)
        arr = np.asarray([(i, m0) for _, i, m0 in work], np.int32).reshape(-1)
        batch.extra[key] = (torch.from_numpy(arr).to(device), len(work))
    return batch.extra[key]


def latent_attention(q_lat, q_rot, pool, batch, rank, scale, path=None,
                     window=0, sink=None, splits=None):
    """``path`` forces "mfma" or "exact" and ``splits`` the number of key
    splits of the tile kernel (tests, tuning); default chooses by size.
    ``q_rot`` is None when rows hold no rotated part."""
    H, T, r = q_lat.shape
    rot = 0 if q_rot is None else q_rot.shape[2]
    assert r == rank and T == batch.n_tokens and window >= 0
    assert pool.shape[-1] == rank + rot and pool.shape[1] == batch.block_size
    assert q_lat.dtype == pool.dtype and pool.is_contiguous()
    if rot:
        assert q_rot.shape[:2] == (T, H) and q_rot.dtype == pool.dtype
        assert q_rot.is_contiguous()
    if sink is not None:
        assert sink.numel() == H
        sink = _f32(sink).contiguous()
    q_lat = q_lat.contiguous()
    lib = load("latent")
    out = torch.empty_like(q_lat)
    reach = min(batch.max_ctx, window) if window > 0 else batch.max_ctx
    mfma = q_lat.dtype == torch.bfloat16 and \
        lib.dsv_latent_attn_mfma_ok(_i(rank), _i(rot)) == 1
    if path is None:
        path = "mfma" if mfma else "exact"
    if path == "mfma":
        assert mfma, "the MFMA kernel is bf16 and bounded in rank"
        rows = lib.dsv_latent_attn_mfma_rows(_i(rank), _i(rot))
        work, n = _tile_work(batch, H, rows, q_lat.device)
        # few tiles over long histories (decoding): split the keys so the
        # launch still covers the chip (about one workgroup per CU: every
        # further split writes and re-reads fp32 partial sums of rank + 2
        # numbers per head, which at 64 requests costs more than the shorter
        # key walk saves); partial sums are merged in fp32
        nsplit = 1
        if n < 128:
            nsplit = max(1, min(32, reach // 128, 256 // n))
        if splits is not None:
            nsplit = max(1, min(int(splits), 64))
        part = None
        if nsplit > 1:
            part = torch.empty(T, nsplit, H, rank + 2, dtype=torch.float32,
                               device=q_lat.device)
        _check(lib.dsv_latent_attn_mfma(
            _p(q_lat), _p(q_rot), _p(pool), _p(work), _i(n), _p(batch.cu),
            _p(batch.seq_start), _p(batch.block_table),
            _i(batch.block_table.shape[1]), _i(batch.block_size), _p(out),
            _p(part), _i(T), _i(H), _i(rank), _i(rot), _i(nsplit), _f(scale),
            _i(window), _p(sink), _stream()), "latent_attention(mfma)")
        return out
    kc, nsplit = _attn_plan(batch, q_lat.dtype, rank, rot, reach)
    part = None
    if nsplit > 1:
        part = torch.empty(T, nsplit, H, rank + 2, dtype=torch.float32,
                           device=q_lat.device)
    _check(lib.dsv_latent_attn(
        _p(q_lat), _p(q_rot), _p(pool), _p(batch.tok_seq), _p(batch.tok_pos),
        _p(batch.block_table), _i(batch.block_table.shape[1]),
        _i(batch.block_size), _p(out), _p(part), _i(_dt(q_lat)), _i(T), _i(H),
        _i(rank), _i(rot), _i(kc), _i(nsplit), _f(scale), _i(window),
        _p(sink), _stream()), "latent_attention")
    return out


def gate_merge_heads(o, gate=None):
    H, T, v = o.shape
    assert gate is None or (gate.shape == (T, H)
                            and gate.dtype == torch.float32)
    out = torch.empty(T, H * v, dtype=o.dtype, device=o.device)
    _check(load("latent").dsv_gate_merge(_p(o.contiguous()), _p(gate), _p(out),
                                 _i(_dt(o)), _i(T), _i(H), _i(v), _stream()),
           "gate_merge_heads")
    return out


# ---------------------------------------------------------- feed-forward
def xielu(z, pq):
    z = z.contiguous()
    out = torch.empty_like(z)
    _check(load().dsv_xielu(_p(z), _p(_f32(pq)), _p(out), _i(_dt(z)),
                            _l(z.numel()), _stream()), "xielu")
    return out


def clamped_swiglu(gu, limit):
    gu = gu.contiguous()
    F = gu.shape[-1] // 2
    rows = gu.numel() // (2 * F)
    out = torch.empty(gu.shape[:-1] + (F,), dtype=gu.dtype, device=gu.device)
    _check(load().dsv_clamped_swiglu(_p(gu), _p(out), _i(_dt(gu)), _l(rows),
                                     _i(F), _f(limit), _stream()),
           "clamped_swiglu")
    return out


def moe_combine(y, inv, weight, shared=None, shared_gate=None):
    T, top = inv.shape
    C = y.shape[1]
    assert y.dim() == 2 and y.is_contiguous() and weight.shape == (T, top)
    assert inv.dtype == torch.int64 and weight.dtype == torch.float32
    if shared is not None:
        assert shared.shape == (T, C) and shared_gate.numel() == T
        assert shared.dtype == y.dtype == shared_gate.dtype
    out = torch.empty(T, C, dtype=y.dtype, device=y.device)
    _check(load().dsv_moe_combine(
        _p(y), _l(y.shape[0]), _p(inv.contiguous()), _p(weight.contiguous()),
        _p(None if shared is None else shared.contiguous()),
        _p(None if shared is None else shared_gate.contiguous()), _p(out),
        _i(_dt(y)), _i(T), _i(top), _i(C), _stream()), "moe_combine")
    return out


def topk_softmax(logits, top):
    T, E = logits.shape
    assert logits.dtype == torch.float32 and 1 <= top <= E
    idx = torch.empty(T, top, dtype=torch.int64, device=logits.device)
    w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    _check(load().dsv_topk_softmax(_p(logits.contiguous()), _p(idx), _p(w),
                                   _i(T), _i(E), _i(top), _stream()),
           "topk_softmax")
    return idx, w


# ------------------------------------------------- layer norm, embedding
def layer_norm_add(x, y, weight, bias, eps, out_dtype=None):
    """x += layer_norm(y) in place; returns the new x rounded to
    ``out_dtype`` (x itself for fp32 / None)."""
    T, C = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert y.shape == x.shape and weight.numel() == C and bias.numel() == C
    y = y.contiguous()
    copy = None
    if out_dtype not in (None, torch.float32):
        copy = torch.empty(T, C, dtype=out_dtype, device=x.device)
    _check(load().dsv_layer_norm(
        _p(y), _i(_dt(y)), _p(None), _p(_f32(weight)), _p(_f32(bias)), _p(x),
        _p(copy), _i(0 if copy is None else _DT[out_dtype]), _i(1), _i(T),
        _i(C), _f(eps), _stream()), "layer_norm_add")
    return x if copy is None else copy


def layer_norm_rows(x, weight, bias, eps, out_dtype, index=None):
    rows = x.shape[0] if index is None else index.numel()
    C = x.shape[1]
    assert weight.numel() == C and bias.numel() == C
    out = torch.empty(rows, C, dtype=out_dtype, device=x.device)
    if index is not None:
        index = index.to(torch.int64).contiguous()
    _check(load().dsv_layer_norm(
        _p(x), _i(_dt(x)), _p(index), _p(_f32(weight)), _p(_f32(bias)),
        _p(None), _p(out), _i(_DT[out_dtype]), _i(0), _i(rows), _i(C),
        _f(eps), _stream()), "layer_norm_rows")
    return out


def embed_rows(table, ids, scale, out_dtype=torch.float32, add_table=None,
               add_ids=None):
    assert table.is_contiguous() and table.dim() == 2
    ids = ids.to(torch.int64).contiguous()
    if add_table is not None:
        assert add_table.is_contiguous() and add_table.dtype == table.dtype
        assert add_table.shape[1] == table.shape[1]
        add_ids = add_ids.to(torch.int64).contiguous()
        assert add_ids.numel() == ids.numel()
    out = torch.empty(ids.numel(), table.shape[1], dtype=torch.float32,
                      device=table.device)
    _check(load().dsv_embed_rows(_p(table), _i(_dt(table)), _p(ids),
                                 _p(add_table), _p(add_ids), _p(out),
                                 _i(ids.numel()), _i(table.shape[1]),
                                 _f(scale), _stream()), "embed_rows")
    return out if out_dtype == torch.float32 else out.to(out_dtype)


def pair_hash_rows(ids, batch, prev, mul_prev, mul_cur, buckets):
    T = ids.numel()
    assert T == batch.n_tokens and ids.dtype == torch.int64
    assert prev.dtype == torch.int64 and prev.dim() == 1
    ids = ids.contiguous()
    rows = torch.empty(T, dtype=torch.int64, device=ids.device)
    _check(load().dsv_pair_hash_rows(
        _p(ids), _p(batch.cu), _p(batch.seq_slot), _p(batch.tok_seq),
        _p(batch.tok_pos), _p(prev), _p(rows), _i(T), _i(batch.n_seqs),
        _l(mul_prev), _l(mul_cur), _l(buckets), _stream()), "pair_hash_rows")
    return rows


def glu(gu, act):
    gu = gu.contiguous()
    F = gu.shape[-1] // 2
    rows = gu.numel() // (2 * F)
    out = torch.empty(gu.shape[:-1] + (F,), dtype=gu.dtype, device=gu.device)
    _check(load().dsv_glu(_p(gu), _p(out), _i(_dt(gu)), _l(rows), _i(F),
                          _i(act), _stream()), "glu")
    return out


def grouped_sigmoid_topk(logits, correction, top, groups, keep):
    return grouped_topk(logits, correction, top, groups, keep, "sigmoid",
                        "top2", False, 1.0)


def grouped_topk(logits, correction, top, groups, keep, score, group_score,
                 renorm, scale):
    T, E = logits.shape
    assert logits.dtype == torch.float32 and correction.numel() == E
    idx = torch.empty(T, top, dtype=torch.int64, device=logits.device)
    w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    _check(load().dsv_grouped_topk(
        _p(logits.contiguous()), _p(_f32(correction).contiguous()), _p(idx),
        _p(w), _i(T), _i(E), _i(top), _i(groups), _i(keep),
        _i(("sigmoid", "softmax").index(score)),
        _i(("top2", "max").index(group_score)), _i(1 if renorm else 0),
        _f(scale), _stream()), "grouped_topk")
    return idx, w


# ------------------------------------------------------ windowed attention
def _seq():
    lib = load("seq")
    lib.dsv_window_attn_lds.restype = ctypes.c_int64
    return lib


def _rows_ok(t):
    """A 2-d operand whose rows are contiguous (a column slice is fine)."""
    assert t.is_cuda and t.dim() == 2 and t.stride(1) == 1
    return t


def _vp(t):
    """Pointer of a view whose rows are contiguous."""
    return ctypes.c_void_p(t.data_ptr())


def attn_prep(proj, batch, pool, q_norm_w, k_norm_w, eps, heads, kv_heads,
              dim, vdim, rot_dims, cos, sin, own_kv=True, norm="whole",
              layout="interleaved", v_unit_eps=None):
    T = proj.shape[0]
    _rows_ok(proj)
    assert proj.dtype == pool.dtype and T == batch.n_tokens
    assert pool.shape[-1] == kv_heads * (dim + vdim) and pool.is_contiguous()
    assert rot_dims % 2 == 0 and rot_dims <= dim
    if rot_dims:
        assert cos.shape[1] == rot_dims // 2 and cos.shape[0] >= batch.max_ctx
        assert cos.dtype == torch.float32 and sin.shape == cos.shape
    q = torch.empty(T, heads, dim, dtype=proj.dtype, device=proj.device)
    if norm == "whole" and layout == "interleaved" and v_unit_eps is None:
        assert proj.is_contiguous() and q_norm_w.numel() == heads * dim
        if own_kv:
            assert k_norm_w.numel() == kv_heads * dim
        _check(_seq().dsv_attn_prep(
            _p(proj), _i(proj.shape[1]), _p(_f32(q_norm_w)),
            _p(_f32(k_norm_w) if own_kv else None), _p(batch.tok_pos),
            _p(batch.tok_row), _p(cos), _p(sin), _p(pool), _p(q),
            _i(_dt(proj)), _i(T), _i(heads), _i(kv_heads), _i(dim), _i(vdim),
            _i(rot_dims), _i(1 if own_kv else 0), _f(eps), _stream()),
            "attn_prep")
        return q
    if norm == "whole":
        raise NotImplementedError(
            "whole-projection norms come with interleaved rotation and plain "
            "values only")
    if norm == "head":
        assert q_norm_w.numel() == dim
        assert not own_kv or k_norm_w.numel() == dim
    _check(_seq().dsv_attn_prep_heads(
        _vp(proj), _i(proj.stride(0)),
        _p(_f32(q_norm_w) if norm == "head" else None),
        _p(_f32(k_norm_w) if norm == "head" and own_kv else None),
        _p(batch.tok_pos), _p(batch.tok_row), _p(cos if rot_dims else None),
        _p(sin if rot_dims else None), _p(pool), _p(q), _i(_dt(proj)), _i(T),
        _i(heads), _i(kv_heads), _i(dim), _i(vdim), _i(rot_dims),
        _i(1 if own_kv else 0), _i(2 if norm == "head" else 0),
        _i(1 if layout == "half" else 0), _f(eps),
        _f(-1.0 if v_unit_eps is None else v_unit_eps), _stream()),
        "attn_prep_heads")
    return q


def _window_tile_work(batch, kv_heads, rep, tile_rows, device):
    """[(sequence, key/value head, first row)] over every sequence's
    count*rep rows per key/value head, late tiles first."""
    key = ("window_tiles", kv_heads, rep, tile_rows)
    if key not in batch.extra:
        import numpy as np
        seqs, firsts, ends = [], [], []
        for i, (st, c) in enumerate(zip(batch.starts, batch.counts)):
            m0 = np.arange(0, c * rep, tile_rows, dtype=np.int32)
            seqs.append(np.full(m0.shape, i, np.int32))
            firsts.append(m0)
            ends.append(st + (m0 + tile_rows) // rep)
        seqs, firsts, ends = (np.concatenate(a) for a in (seqs, firsts, ends))
        order = np.argsort(-ends, kind="stable")
        n = order.size
        work = np.empty((kv_heads, n, 3), np.int32)
        work[:, :, 0] = seqs[order]
        work[:, :, 1] = np.arange(kv_heads, dtype=np.int32)[:, None]
        work[:, :, 2] = firsts[order]
        work = np.ascontiguousarray(work.transpose(1, 0, 2)).reshape(-1)
        batch.extra[key] = (torch.from_numpy(work).to(device), n * kv_heads)
    return batch.extra[key]


def window_attention(q, pool, batch, kv_heads, dim, vdim, scale, window=0,
                     keep_first=0, path=None, chunk=0, softcap=0.0,
                     out_scale=1.0, out=None):
    """``path`` forces "mfma" or "exact" (tests); default: the tile kernel for
    bf16 at head sizes it covers (prompt portions and, with split keys, single
    tokens), the exact kernel otherwise (fp32)."""
    T, H, d = q.shape
    assert d == dim and T == batch.n_tokens and q.is_contiguous()
    assert pool.shape[1] == batch.block_size and pool.is_contiguous()
    assert q.dtype == pool.dtype and H % kv_heads == 0
    assert pool.shape[-1] == kv_heads * (dim + vdim)
    assert not (window > 0 and chunk > 0)
    lib = _seq()
    dt = _dt(q)
    reach = batch.max_ctx
    if window > 0:
        reach = min(reach, window + keep_first)
    elif chunk > 0:
        reach = min(reach, chunk + keep_first)
    if out is None:
        out = torch.empty(T, H * vdim, dtype=q.dtype, device=q.device)
    assert out.shape == (T, H * vdim) and out.stride(1) == 1
    assert out.dtype == q.dtype and out.is_cuda
    ld_out = out.stride(0)
    mfma = q.dtype == torch.bfloat16 and \
        lib.dsv_window_attn_mfma_ok(_i(dim), _i(vdim)) == 1
    if path is None:
        path = "mfma" if mfma else "exact"
    if path == "mfma":
        assert mfma, "the MFMA kernel is bf16 with head sizes up to 256"
        rep = H // kv_heads
        work, n = _window_tile_work(batch, kv_heads, rep,
                                    lib.dsv_window_attn_mfma_rows(), q.device)
        # few tiles over long visible ranges (decoding): split the keys so
        # the launch still covers the chip; partial sums are merged in fp32
        nsplit = 1
        if n < 256:
            nsplit = max(1, min(32, reach // 64, 1024 // n))
        part = None
        if nsplit > 1:
            part = torch.empty(T, nsplit, H, vdim + 2, dtype=torch.float32,
                               device=q.device)
        _check(lib.dsv_window_attn_mfma(
            _p(q), _p(pool), _p(work), _i(n), _p(batch.cu),
            _p(batch.seq_start), _p(batch.block_table),
            _i(batch.block_table.shape[1]), _i(batch.block_size), _vp(out),
            _i(ld_out), _p(part), _i(T), _i(H), _i(kv_heads), _i(dim),
            _i(vdim), _i(nsplit), _f(scale), _i(window), _i(keep_first),
            _i(chunk), _f(softcap), _f(out_scale), _stream()),
            "window_attention(mfma)")
        return out
    kc = 64
    while kc > 4 and lib.dsv_window_attn_lds(dt, dim, vdim, kc) > 60 * 1024:
        kc //= 2
    # few tokens over a long visible range (decoding): split the keys so the
    # launch still covers the chip; partial sums are merged in fp32
    nsplit = 1
    if T * kv_heads <= 128:
        nsplit = max(1, min(32, reach // (4 * kc),
                            1024 // max(1, T * kv_heads)))
    part = None
    if nsplit > 1:
        part = torch.empty(T, nsplit, H, vdim + 2, dtype=torch.float32,
                           device=q.device)
    _check(lib.dsv_window_attn(
        _p(q), _p(pool), _p(batch.tok_seq), _p(batch.tok_pos),
        _p(batch.block_table), _i(batch.block_table.shape[1]),
        _i(batch.block_size), _vp(out), _i(ld_out), _p(part), _i(dt), _i(T),
        _i(H), _i(kv_heads), _i(dim), _i(vdim), _i(kc), _i(nsplit), _f(scale),
        _i(window), _i(keep_first), _i(chunk), _f(softcap), _f(out_scale),
        _stream()), "window_attention")
    return out


# ------------------------------------------------------ linear recurrences
def delta_prep(proj, batch, conv_w, conv_state, a_log, dt_bias, kv_heads,
               heads, dim, vdim, beta_col=None, a_col=None):
    T = proj.shape[0]
    taps = conv_w.shape[1]
    C = 2 * kv_heads * dim + heads * vdim
    if beta_col is None:
        beta_col = C + heads * vdim
    if a_col is None:
        a_col = beta_col + heads
    assert 0 <= beta_col <= proj.shape[1] - heads
    assert a_col < 0 or a_col <= proj.shape[1] - heads
    assert proj.is_contiguous() and T == batch.n_tokens
    assert conv_w.dtype == proj.dtype == conv_state.dtype
    assert conv_w.is_contiguous() and conv_w.shape[0] == C
    assert conv_state.shape[1:] == (taps - 1, C)
    assert conv_state.stride(2) == 1 and (taps == 1
                                          or conv_state.stride(1) == C)
    dev = proj.device
    f32 = dict(dtype=torch.float32, device=dev)
    q = torch.empty(T, kv_heads, dim, **f32)
    k = torch.empty(T, kv_heads, dim, **f32)
    v = torch.empty(T, heads, vdim, **f32)
    beta = torch.empty(T, heads, **f32)
    decay = torch.empty(T, heads, **f32) if a_col >= 0 else None
    _check(_seq().dsv_delta_prep(
        _p(proj), _i(proj.shape[1]), _p(conv_w),
        ctypes.c_void_p(conv_state.data_ptr()), _l(conv_state.stride(0)),
        _p(batch.cu), _p(batch.seq_slot), _p(batch.seq_start),
        _p(batch.tok_seq), _p(batch.tok_pos),
        _p(_f32(a_log) if a_col >= 0 else None),
        _p(_f32(dt_bias) if a_col >= 0 else None), _p(q), _p(k), _p(v),
        _p(beta), _p(decay),
        _i(_dt(proj)), _i(T), _i(batch.n_seqs), _i(kv_heads), _i(heads),
        _i(dim), _i(vdim), _i(taps), _i(beta_col), _i(a_col), _stream()),
        "delta_prep")
    return q, k, v, beta, decay


def softplus_decay(z, bias, a_log, heads):
    T, C = z.shape
    _rows_ok(z)
    assert C % heads == 0 and bias.numel() == C and a_log.numel() == heads
    out = torch.empty(T, heads, C // heads, dtype=torch.float32,
                      device=z.device)
    _check(_seq().dsv_softplus_decay(
        _vp(z), _i(z.stride(0)), _p(_f32(bias).contiguous()),
        _p(_f32(a_log).contiguous()), _p(out), _i(_dt(z)), _l(T), _i(heads),
        _i(C // heads), _stream()), "softplus_decay")
    return out


def sigmoid_pow(z, bias, inv_tau):
    z = z.contiguous()
    C = z.shape[-1]
    assert bias.numel() == C
    out = torch.empty(z.shape, dtype=torch.float32, device=z.device)
    _check(_seq().dsv_sigmoid_pow(_p(z), _p(_f32(bias)), _p(out), _i(_dt(z)),
                                  _l(z.numel()), _i(C), _f(inv_tau),
                                  _stream()), "sigmoid_pow")
    return out


def _heads_view(t):
    """[T, n, d] whose heads are side by side in a row: row stride."""
    assert t.is_cuda and t.stride(2) == 1 and t.stride(1) == t.shape[2]
    return ctypes.c_void_p(t.data_ptr()), _i(t.stride(0))


def linear_scan(q, k, v, decay, beta, state, batch, q_scale=1.0):
    T, G, dim = q.shape
    H, vdim = v.shape[1], v.shape[2]
    assert q.dtype == k.dtype == v.dtype and k.shape == q.shape
    assert T == batch.n_tokens and v.shape[0] == T
    assert state.dtype == torch.float32 and state.is_contiguous()
    assert state.shape[1:] == (H, dim, vdim)
    assert decay.dtype == torch.float32 and decay.is_contiguous()
    channel = decay.dim() == 3
    assert decay.shape == ((T, H, dim) if channel else (T, H))
    if beta is not None:
        assert beta.shape == (T, H) and beta.dtype == torch.float32
        beta = beta.contiguous()
    out = torch.empty(T, H, vdim, dtype=torch.float32, device=q.device)
    (qp, ldq), (kp, ldk), (vp, ldv) = (_heads_view(t) for t in (q, k, v))
    _check(_seq().dsv_linear_scan(
        qp, ldq, kp, ldk, vp, ldv, _p(decay), _i(1 if channel else 0),
        _p(beta), _p(state), _p(batch.cu), _p(batch.seq_slot), _p(out),
        _i(_dt(q)), _i(batch.n_seqs), _i(G), _i(H), _i(dim), _i(vdim),
        _f(q_scale), _stream()), "linear_scan")
    return out


def head_norm_gate(o, weight, gate, eps, out_dtype, act="silu"):
    T, H, vdim = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous()
    assert weight.numel() == vdim and gate.shape == (T, H * vdim)
    assert gate.dtype == out_dtype
    _rows_ok(gate)
    out = torch.empty(T, H * vdim, dtype=out_dtype, device=o.device)
    _check(_seq().dsv_head_norm_gate(
        _p(o), _p(_f32(weight)), ctypes.c_void_p(gate.data_ptr()),
        _i(gate.stride(0)), _p(out), _i(_DT[out_dtype]), _i(T), _i(H),
        _i(vdim), _f(eps), _i(("silu", "sigmoid").index(act)), _stream()),
        "head_norm_gate")
    return out


# ------------------------------------- state-space prologues and epilogue
def conv_silu_ragged(x, conv_w, state, batch, bias=None, out_dtype=None):
    T, C = x.shape
    taps = conv_w.shape[1]
    out_dtype = out_dtype or torch.float32
    _rows_ok(x)
    assert T == batch.n_tokens and out_dtype in (torch.float32, x.dtype)
    assert conv_w.dtype == x.dtype == state.dtype
    assert conv_w.is_contiguous() and conv_w.shape[0] == C
    assert state.shape[1:] == (taps - 1, C)
    assert state.stride(2) == 1 and (taps == 1 or state.stride(1) == C)
    out = torch.empty(T, C, dtype=out_dtype, device=x.device)
    _check(_seq().dsv_conv_silu(
        _vp(x), _i(x.stride(0)), _p(conv_w),
        _p(None if bias is None else _f32(bias)), _vp(state),
        _l(state.stride(0)), _p(batch.cu), _p(batch.seq_slot),
        _p(batch.seq_start), _p(batch.tok_seq), _p(batch.tok_pos), _p(out),
        _i(_dt(x)), _i(0 if out_dtype == torch.float32 else 1), _i(T),
        _i(batch.n_seqs), _i(C), _i(taps), _stream()), "conv_silu")
    return out


def ssd_prep(proj, batch, conv_w, conv_b, conv_state, a_log, dt_bias, heads,
             groups, state, vdim):
    T = proj.shape[0]
    taps = conv_w.shape[1]
    inner, gn = heads * vdim, groups * state
    C = inner + 2 * gn
    _rows_ok(proj)
    assert T == batch.n_tokens and proj.shape[1] == 2 * inner + 2 * gn + heads
    assert conv_w.dtype == proj.dtype == conv_state.dtype
    assert conv_w.is_contiguous() and conv_w.shape[0] == C
    assert conv_b.numel() == C and a_log.numel() == heads
    assert dt_bias.numel() == heads
    assert conv_state.shape[1:] == (taps - 1, C)
    assert conv_state.stride(2) == 1 and (taps == 1
                                          or conv_state.stride(1) == C)
    f32 = dict(dtype=torch.float32, device=proj.device)
    x = torch.empty(T, heads, vdim, **f32)
    v = torch.empty(T, heads, vdim, **f32)
    Bk = torch.empty(T, groups, state, **f32)
    Cq = torch.empty(T, groups, state, **f32)
    decay = torch.empty(T, heads, **f32)
    _check(_seq().dsv_ssd_prep(
        _vp(proj), _i(proj.stride(0)), _p(conv_w), _p(_f32(conv_b)),
        _vp(conv_state), _l(conv_state.stride(0)), _p(batch.cu),
        _p(batch.seq_slot), _p(batch.seq_start), _p(batch.tok_seq),
        _p(batch.tok_pos), _p(_f32(a_log)), _p(_f32(dt_bias)), _p(x), _p(v),
        _p(Bk), _p(Cq), _p(decay), _i(_dt(proj)), _i(T), _i(batch.n_seqs),
        _i(heads), _i(vdim), _i(groups), _i(state), _i(taps), _stream()),
        "ssd_prep")
    return Cq, Bk, v, x, decay


def gate_group_norm(o, x, skip, gate, weight, parts, eps, out_dtype):
    T, H, vdim = o.shape
    n = H * vdim
    assert o.dtype == torch.float32 and o.is_contiguous()
    assert x.dtype == torch.float32 and x.is_contiguous() and x.shape == o.shape
    assert skip.numel() == H and weight.numel() == n and n % parts == 0
    assert gate.shape == (T, n) and gate.dtype == out_dtype
    _rows_ok(gate)
    out = torch.empty(T, n, dtype=out_dtype, device=o.device)
    _check(_seq().dsv_gate_group_norm(
        _p(o), _p(x), _p(_f32(skip)), _vp(gate), _i(gate.stride(0)),
        _p(_f32(weight)), _p(out), _i(_DT[out_dtype]), _i(T), _i(H), _i(vdim),
        _i(parts), _f(eps), _stream()), "gate_group_norm")
    return out


def selective_scan(x, dt_pre, dt_bias, a_log, B, C, skip, z, state, batch,
                   out_scale, out):
    T, ch = x.shape
    n = a_log.shape[1]
    for t in (x, B, C, z, out):
        _rows_ok(t)
    assert x.dtype == B.dtype == C.dtype == z.dtype == out.dtype
    assert B.stride(0) == C.stride(0) and T == batch.n_tokens
    assert dt_pre.is_contiguous() and dt_pre.dtype == torch.float32
    assert state.dtype == torch.float32 and state.is_contiguous()
    assert state.shape[1:] == (ch, n) and a_log.shape == (ch, n)
    assert dt_bias.numel() == ch and skip.numel() == ch
    lib = _seq()
    if n > lib.dsv_selective_scan_max_state():
        raise ValueError("selective scan: state size beyond the kernel's")
    _check(lib.dsv_selective_scan(
        _vp(x), _i(x.stride(0)), _p(dt_pre), _p(_f32(dt_bias)),
        _p(_f32(a_log).contiguous()), _vp(B), _vp(C), _i(B.stride(0)),
        _p(_f32(skip)), _vp(z), _i(z.stride(0)), _p(state), _p(batch.cu),
        _p(batch.seq_slot), _vp(out), _i(out.stride(0)), _i(_dt(x)),
        _i(batch.n_seqs), _i(ch), _i(n), _f(out_scale), _stream()),
        "selective_scan")
    return out


# --------------------------------------- weighted RMS norm, gated residual
def rms_norm_rows(x, weight, eps, out_dtype, index=None, one_plus=False):
    rows = x.shape[0] if index is None else index.numel()
    C = x.shape[1]
    _rows_ok(x)
    assert weight.numel() == C
    out = torch.empty(rows, C, dtype=out_dtype, device=x.device)
    if index is not None:
        index = index.to(torch.int64).contiguous()
    _check(load().dsv_rms_norm_rows(
        _vp(x), _i(_dt(x)), _i(x.stride(0)), _p(index), _p(_f32(weight)),
        _p(out), _i(_DT[out_dtype]), _i(rows), _i(C), _f(eps),
        _i(1 if one_plus else 0), _stream()), "rms_norm_rows")
    return out


def scaled_add(x, s1, y1, s2, y2, extra, w1, w2, eps, out_dtype):
    """x += s1*y1 (+ s2*y2) (+ extra) in place; returns (h1, h2): the RMS
    norms of the new x under w1 / w2 (None where no weight is given)."""
    T, C = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    dt = _dt(x)
    if y1 is not None:
        y1 = y1.contiguous()
        assert y1.shape == (T, C) and s1.numel() == C
        dt = _dt(y1)
    if y2 is not None:
        y2 = y2.contiguous()
        assert y1 is not None and y2.shape == (T, C) and s2.numel() == C
        assert y2.dtype == y1.dtype
    if extra is not None:
        assert extra.shape == (T, C) and extra.dtype == torch.float32
        extra = extra.contiguous()
    h1 = h2 = None
    out_dtype = out_dtype or torch.float32
    if w1 is not None:
        assert w1.numel() == C
        h1 = torch.empty(T, C, dtype=out_dtype, device=x.device)
    if w2 is not None:
        assert w1 is not None and w2.numel() == C
        h2 = torch.empty(T, C, dtype=out_dtype, device=x.device)
    f = lambda t: None if t is None else _f32(t).contiguous()
    _check(load().dsv_scaled_add(
        _p(x), _p(f(s1) if y1 is not None else None), _p(y1),
        _p(f(s2) if y2 is not None else None), _p(y2), _p(extra), _p(f(w1)),
        _p(f(w2)), _p(h1), _p(h2), _i(dt), _i(_DT[out_dtype]), _i(T), _i(C),
        _f(eps), _stream()), "scaled_add")
    return h1, h2


def gated_add(x, g1, y1, g2, y2, norm_weight, eps, out_dtype, one_plus):
    T, C = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert g1.shape == (T, C) and y1.shape == (T, C)
    _rows_ok(g1)
    y1 = y1.contiguous()
    assert g1.dtype == y1.dtype
    if y2 is not None:
        _rows_ok(g2)
        y2 = y2.contiguous()
        assert g2.shape == (T, C) and y2.shape == (T, C)
        assert g2.dtype == y2.dtype == y1.dtype
        assert g2.stride(0) == g1.stride(0)
    h = None
    if norm_weight is not None:
        out_dtype = out_dtype or torch.float32
        assert norm_weight.numel() == C
        h = torch.empty(T, C, dtype=out_dtype, device=x.device)
    _check(load().dsv_gated_add(
        _p(x), _vp(g1), _p(None) if y2 is None else _vp(g2),
        _i(g1.stride(0)), _p(y1), _p(y2),
        _p(None if norm_weight is None else _f32(norm_weight)), _p(h),
        _i(_dt(y1)), _i(0 if h is None else _DT[h.dtype]), _i(T), _i(C),
        _f(eps), _i(1 if one_plus else 0), _stream()), "gated_add")
    return h


def act_rows(z, act):
    T, F = z.shape
    _rows_ok(z)
    out = torch.empty(T, F, dtype=z.dtype, device=z.device)
    _check(load().dsv_act_rows(_vp(z), _i(z.stride(0)), _p(out), _i(_dt(z)),
                               _l(T), _i(F), _i(act), _stream()), "act_rows")
    return out


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
