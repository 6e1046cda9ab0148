"""Latent (compressed-KV) attention over a paged cache, for ragged batches.

Every token caches ONE row shared by all heads: ``[c ; k_rot]`` with ``c`` the
normed latent (``rank`` numbers) and ``k_rot`` the rotated key part
(``rot`` numbers). Per head the unrotated key is ``W_uk c`` and the value
``W_uv c``; both up-projections are folded into the query and the output
instead of being applied to the cache:

    score(i, j) = ((W_uk^T q_nope_i) . c_j + q_rot_i . k_rot_j) * scale
    out_i       = W_uv (sum_j p_ij c_j)

so the attention kernel is multi-query attention whose key is the cached row
and whose value is its first ``rank`` entries. Scores, softmax and the
weighted sum are fp32. Position i of a sequence sees rows 0..i.

``latent_prep`` finishes the fused input projection of a step: norm of the
latent, rotation of the shared key part and of the queries' rotated parts,
the output gate's sigmoid, and the write of the new rows into the pool.
"""

import torch

from .rope import rope_interleaved_


def _sk():
    from . import serving_kernels
    return serving_kernels


def latent_prep(proj, batch, pool, norm_w, eps, heads, dim, rot, rank,
                rot_dims, cos, sin):
    """proj [T, heads*(dim+rot) + rank + rot + heads] = q | latent | k_rot |
    gate logits. Writes the new rows into ``pool`` ([blocks, bs, rank+rot]).
    Returns q_nope [heads, T, dim] (contiguous), q_rot [T, heads, rot],
    gate [T, heads] fp32."""
    if proj.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.latent_prep(proj, batch, pool, norm_w, eps, heads, dim, rot,
                              rank, rot_dims, cos, sin)
    T = proj.shape[0]
    nq = heads * (dim + rot)
    q = proj[:, :nq].reshape(T, heads, dim + rot)
    lat = proj[:, nq:nq + rank].float()
    c = lat * torch.rsqrt(lat.pow(2).mean(-1, keepdim=True) + eps) \
        * norm_w.float()
    kr = proj[:, nq + rank:nq + rank + rot].clone()
    rope_interleaved_(kr, batch.tok_pos, cos, sin, rot_dims)
    q_rot = q[..., dim:].clone()
    rope_interleaved_(q_rot, batch.tok_pos, cos, sin, rot_dims)
    rows = torch.cat([c.to(pool.dtype), kr.to(pool.dtype)], -1)
    pool.view(-1, rank + rot)[batch.tok_row.long()] = rows
    gate = torch.sigmoid(proj[:, nq + rank + rot:].float())
    q_nope = q[..., :dim].transpose(0, 1).contiguous()
    return q_nope, q_rot, gate


def latent_attention(q_lat, q_rot, pool, batch, rank, scale):
    """q_lat [heads, T, rank], q_rot [T, heads, rot]; pool holds every
    sequence's rows INCLUDING this step's. Returns [heads, T, rank]."""
    if q_lat.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.latent_attention(q_lat, q_rot, pool, batch, rank, scale)
    bs = batch.block_size
    rows = pool.view(-1, pool.shape[-1])
    out = torch.empty_like(q_lat)
    at = 0
    for i, (st, cnt) in enumerate(zip(batch.starts, batch.counts)):
        L = st + cnt
        pos = torch.arange(L, device=q_lat.device)
        ctx = rows[batch.block_table[i].long()[pos // bs] * bs + pos % bs]
        ctx = ctx.float()
        s = torch.einsum("htr,lr->htl", q_lat[:, at:at + cnt].float(),
                         ctx[:, :rank])
        s = s + torch.einsum("thd,ld->htl", q_rot[at:at + cnt].float(),
                             ctx[:, rank:])
        s = s * scale
        qpos = st + torch.arange(cnt, device=q_lat.device)
        s = s.masked_fill(pos[None, None, :] > qpos[None, :, None],
                          float("-inf"))
        p = torch.softmax(s, -1)
        out[:, at:at + cnt] = torch.einsum("htl,lr->htr", p,
                                           ctx[:, :rank]).to(out.dtype)
        at += cnt
    return out


def gate_merge_heads(o, gate):
    """o [heads, T, v], gate [T, heads] fp32 -> [T, heads*v] (o's dtype)."""
    if o.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.gate_merge_heads(o, gate)
    H, T, v = o.shape
    return (o.float().transpose(0, 1) * gate[:, :, None]).to(o.dtype) \
        .reshape(T, H * v)
