"""ctypes front-end of the ragged-batch serving kernels
(csrc/serving/serving_kernels.hip -> deepspeed_amd/ops/_serving.so).

The library has a plain C ABI, so it builds with one hipcc call in a few
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
SOURCE = os.path.join(_HERE, "csrc", "serving", "serving_kernels.hip")
LIBRARY = os.path.join(_HERE, "_serving.so")
HIPCC_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-shared", "-fPIC"]

_lib = None


def _compile(target):
    hipcc = os.environ.get("HIPCC") or (
        "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc")
        else "hipcc")
    tmp = "%s.%d.tmp" % (target, os.getpid())
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", tmp, SOURCE]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True)
    if r.returncode != 0:
        raise RuntimeError("building the serving kernels failed:\n" + r.stdout)
    os.replace(tmp, target)
    return target


def _fresh(path):
    return os.path.exists(path) and \
        os.path.getmtime(path) >= os.path.getmtime(SOURCE)


def build(force=True):
    """Compile the library in-tree (cross-compiles without a GPU). Returns the
    path of the library to load. Where the tree cannot be written, a copy
    keyed by the source's content goes to the temporary directory instead."""
    if not force and _fresh(LIBRARY):
        return LIBRARY
    if os.access(os.path.dirname(LIBRARY), os.W_OK):
        return _compile(LIBRARY)
    import hashlib
    import tempfile
    with open(SOURCE, "rb") as f:
        tag = hashlib.sha1(f.read()).hexdigest()[:16]
    alt = os.path.join(tempfile.gettempdir(), "ds_amd_serving_%s.so" % tag)
    return alt if os.path.exists(alt) else _compile(alt)


def load():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build(force=False))
        _lib.dsv_latent_attn_lds.restype = ctypes.c_int64
    return _lib


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
def latent_prep(proj, batch, pool, norm_w, eps, heads, dim, rot, rank,
                rot_dims, cos, sin):
    T = proj.shape[0]
    assert proj.is_contiguous() and proj.dtype == pool.dtype
    assert proj.shape[1] == heads * (dim + rot) + rank + rot + heads
    assert pool.shape[-1] == rank + rot and T == batch.n_tokens
    assert rot_dims % 2 == 0 and rot_dims <= rot
    assert cos.shape[1] == rot_dims // 2 and cos.shape[0] >= batch.max_ctx
    assert cos.dtype == torch.float32 and sin.shape == cos.shape
    dev, dt = proj.device, proj.dtype
    q_nope = torch.empty(heads, T, dim, dtype=dt, device=dev)
    q_rot = torch.empty(T, heads, rot, dtype=dt, device=dev)
    gate = torch.empty(T, heads, dtype=torch.float32, device=dev)
    _check(load().dsv_latent_prep(
        _p(proj), _i(proj.shape[1]), _p(_f32(norm_w)), _p(batch.tok_pos),
        _p(batch.tok_row), _p(cos), _p(sin), _p(pool), _p(q_nope), _p(q_rot),
        _p(gate), _i(_dt(proj)), _i(T), _i(heads), _i(dim), _i(rot), _i(rank),
        _i(rot_dims), _f(eps), _stream()), "latent_prep")
    return q_nope, q_rot, gate


def _attn_plan(batch, dtype, rank, rot):
    """Key-chunk length that fits LDS, and the number of key splits: few
    tokens over a long history are split so the launch still fills the chip."""
    lib = load()
    dt = _DT[dtype]
    kc = 64
    while kc > 4 and lib.dsv_latent_attn_lds(dt, rank, rot, kc) > 60 * 1024:
        kc //= 2
    nsplit = 1
    if batch.n_tokens <= 128:
        nsplit = max(1, min(32, batch.max_ctx // (4 * kc),
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


def latent_attention(q_lat, q_rot, pool, batch, rank, scale, path=None):
    """``path`` forces "mfma" or "exact" (tests); default chooses by size."""
    H, T, r = q_lat.shape
    rot = q_rot.shape[2]
    assert r == rank and q_rot.shape[:2] == (T, H) and T == batch.n_tokens
    assert pool.shape[-1] == rank + rot and pool.shape[1] == batch.block_size
    assert q_lat.dtype == pool.dtype == q_rot.dtype
    assert q_rot.is_contiguous() and pool.is_contiguous()
    q_lat = q_lat.contiguous()
    lib = load()
    out = torch.empty_like(q_lat)
    mfma = q_lat.dtype == torch.bfloat16 and \
        lib.dsv_latent_attn_mfma_ok(_i(rank), _i(rot)) == 1
    if path is None:
        path = "mfma" if mfma else "exact"
    if path == "mfma":
        assert mfma, "the MFMA kernel is bf16 and bounded in rank"
        rows = lib.dsv_latent_attn_mfma_rows(_i(rank), _i(rot))
        work, n = _tile_work(batch, H, rows, q_lat.device)
        # few tiles over long histories (decoding): split the keys so the
        # launch still covers the chip; partial sums are merged in fp32
        nsplit = 1
        if n < 128:
            nsplit = max(1, min(32, batch.max_ctx // 128, 512 // n))
        part = None
        if nsplit > 1:
            part = torch.empty(T, nsplit, H, rank + 2, dtype=torch.float32,
                               device=q_lat.device)
        _check(lib.dsv_latent_attn_mfma(
            _p(q_lat), _p(q_rot), _p(pool), _p(work), _i(n), _p(batch.cu),
            _p(batch.seq_start), _p(batch.block_table),
            _i(batch.block_table.shape[1]), _i(batch.block_size), _p(out),
            _p(part), _i(T), _i(H), _i(rank), _i(rot), _i(nsplit), _f(scale),
            _stream()), "latent_attention(mfma)")
        return out
    kc, nsplit = _attn_plan(batch, q_lat.dtype, rank, rot)
    part = None
    if nsplit > 1:
        part = torch.empty(T, nsplit, H, rank + 2, dtype=torch.float32,
                           device=q_lat.device)
    _check(lib.dsv_latent_attn(
        _p(q_lat), _p(q_rot), _p(pool), _p(batch.tok_seq), _p(batch.tok_pos),
        _p(batch.block_table), _i(batch.block_table.shape[1]),
        _i(batch.block_size), _p(out), _p(part), _i(_dt(q_lat)), _i(T), _i(H),
        _i(rank), _i(rot), _i(kc), _i(nsplit), _f(scale), _stream()),
        "latent_attention")
    return out


def gate_merge_heads(o, gate):
    H, T, v = o.shape
    assert gate.shape == (T, H) and gate.dtype == torch.float32
    out = torch.empty(T, H * v, dtype=o.dtype, device=o.device)
    _check(load().dsv_gate_merge(_p(o.contiguous()), _p(gate), _p(out),
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
    assert y.shape[0] >= T * top and weight.shape == (T, top)
    assert inv.dtype == torch.int64 and weight.dtype == torch.float32
    if shared is not None:
        assert shared.shape == (T, C) and shared_gate.numel() == T
        assert shared.dtype == y.dtype == shared_gate.dtype
    out = torch.empty(T, C, dtype=y.dtype, device=y.device)
    _check(load().dsv_moe_combine(
        _p(y), _p(inv.contiguous()), _p(weight.contiguous()),
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


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
