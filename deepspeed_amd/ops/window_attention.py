"""Multi-head attention over paged K/V rows with a sliding window that also
keeps a sequence's first tokens, for ragged batches.

Every token caches ONE row per stream: ``[k (G x dim) ; v (G x vdim)]`` for the
G key/value heads; query head h reads key/value head ``h // (H / G)``. Position
i of a sequence sees position j when ``j <= i`` and (``i - j < window`` or
``j < keep_first``); kept tokens stay where they are (their rows were rotated
at their true positions). ``window <= 0`` means no window (plain causal).
Scores, softmax and the weighted sum are fp32.

``attn_prep`` finishes a step's fused q|k|v projection: RMS norm of the WHOLE
query projection (all heads at once, one weight per coordinate) and of the
whole key projection, interleaved rotation of the first ``rot_dims``
coordinates of every head, and the write of the new rows into the pool. A
layer that borrows another layer's rows passes ``own_kv=False``: its
projection holds queries only and nothing is written.
"""

import torch

from .rope import rope_interleaved_


def _sk():
    from . import serving_kernels
    return serving_kernels


def _rms_all(x, w, eps):
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()


def attn_prep(proj, batch, pool, q_norm_w, k_norm_w, eps, heads, kv_heads,
              dim, vdim, rot_dims, cos, sin, own_kv=True):
    """proj [T, heads*dim (+ kv_heads*dim + kv_heads*vdim)] = q | k | v.
    Returns q [T, heads, dim] in proj's dtype; with ``own_kv`` the rows
    [k ; v] of this step's tokens are written into ``pool``
    ([blocks, block_size, kv_heads*(dim+vdim)])."""
    T = proj.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    assert proj.shape[1] == nq + (nk + nv if own_kv else 0)
    if proj.is_cuda and _sk().enabled():
        return _sk().attn_prep(proj, batch, pool, q_norm_w, k_norm_w, eps,
                               heads, kv_heads, dim, vdim, rot_dims, cos, sin,
                               own_kv)
    q = _rms_all(proj[:, :nq], q_norm_w, eps).reshape(T, heads, dim)
    rope_interleaved_(q, batch.tok_pos, cos, sin, rot_dims)
    if own_kv:
        k = _rms_all(proj[:, nq:nq + nk], k_norm_w, eps) \
            .reshape(T, kv_heads, dim)
        rope_interleaved_(k, batch.tok_pos, cos, sin, rot_dims)
        rows = torch.cat([k.reshape(T, nk).to(pool.dtype),
                          proj[:, nq + nk:].to(pool.dtype)], -1)
        pool.view(-1, nk + nv)[batch.tok_row.long()] = rows
    return q.to(proj.dtype)


def window_mask(qpos, kpos, window, keep_first):
    """[len(qpos), len(kpos)] bool: which keys each query sees."""
    d = qpos[:, None] - kpos[None, :]
    near = d >= 0
    if window > 0:
        near = near & ((d < window) | (kpos[None, :] < keep_first))
    return near


def window_attention(q, pool, batch, kv_heads, dim, vdim, scale, window=0,
                     keep_first=0, path=None):
    """q [T, heads, dim]; pool holds every sequence's rows INCLUDING this
    step's. Returns [T, heads*vdim] in q's dtype."""
    T, H, _ = q.shape
    assert H % kv_heads == 0 and pool.shape[-1] == kv_heads * (dim + vdim)
    if q.is_cuda and _sk().enabled():
        return _sk().window_attention(q, pool, batch, kv_heads, dim, vdim,
                                      scale, window, keep_first, path)
    bs = batch.block_size
    rows = pool.view(-1, pool.shape[-1])
    out = torch.empty(T, H, vdim, dtype=q.dtype, device=q.device)
    rep = H // kv_heads
    at = 0
    for i, (st, cnt) in enumerate(zip(batch.starts, batch.counts)):
        L = st + cnt
        pos = torch.arange(L, device=q.device)
        ctx = rows[batch.block_table[i].long()[pos // bs] * bs + pos % bs]
        ctx = ctx.float()
        k = ctx[:, :kv_heads * dim].reshape(L, kv_heads, dim) \
            .repeat_interleave(rep, 1)
        v = ctx[:, kv_heads * dim:].reshape(L, kv_heads, vdim) \
            .repeat_interleave(rep, 1)
        s = torch.einsum("thd,lhd->htl", q[at:at + cnt].float(), k) * scale
        see = window_mask(st + torch.arange(cnt, device=q.device), pos,
                          window, keep_first)
        s = s.masked_fill(~see[None], float("-inf"))
        p = torch.softmax(s, -1)
        out[at:at + cnt] = torch.einsum("htl,lhv->thv", p, v).to(q.dtype)
        at += cnt
    return out.reshape(T, H * vdim)
