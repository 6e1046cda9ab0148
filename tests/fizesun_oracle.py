"""Plain, slow Fizesun forward: one function per mechanism, whole sequences,
no cache, no batching. Written directly from the design's equations and used
only as the oracle that the serving path is compared with; it shares no code
with ``deepspeed_amd``.

A model is (cfg, w): ``cfg`` the parsed config dict, ``w`` a dict
name -> float64/float32 tensor. Every function takes and returns tensors of
one sequence, time first.
"""

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is a single number."""
    return rms(x, eps) * g.reshape(())


def causal_taps(h, w):
    """h [S, C], w [C, taps]: out_t = sum_j w[:, j] * h[t - taps + 1 + j]."""
    S, C = h.shape
    taps = w.shape[1]
    out = torch.zeros_like(h)
    for t in range(S):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def with_input_conv(h, w):
    return h + causal_taps(h, w)


def rotate_pairs(v, pos, dims, base):
    """v [..., n]: dimensions (2i, 2i+1), i < dims/2, turned by pos * base^(-2i/dims)."""
    out = v.clone()
    for i in range(dims // 2):
        a = pos * (base ** (-2.0 * i / dims))
        c, s = math.cos(a), math.sin(a)
        u, w_ = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w_ * s
        out[..., 2 * i + 1] = w_ * c + u * s
    return out


def latent_attention(h, w, pre, m, eps):
    """h [S, width] -> [S, width]; m is the layer's 'mixer' dict."""
    S = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    q = (h @ w[pre + "q"].T).reshape(S, H, dn + dr)
    dkv = h @ w[pre + "dkv"].T
    c = rms(dkv[:, :r], eps) * w[pre + "dkv.norm"]
    kr = dkv[:, r:]
    kn = (c @ w[pre + "uk"].T).reshape(S, H, dn)
    val = (c @ w[pre + "uv"].T).reshape(S, H, dv)
    gate = torch.sigmoid(h @ w[pre + "g"].T)                     # [S, H]
    qn, qr = q[..., :dn], q[..., dn:].clone()
    kr = kr.clone()
    for t in range(S):
        qr[t] = rotate_pairs(qr[t], t, rd, base)
        kr[t] = rotate_pairs(kr[t], t, rd, base)
    out = torch.zeros(S, H, dv, dtype=h.dtype)
    for t in range(S):
        for a in range(H):
            s = (kn[: t + 1, a] @ qn[t, a] + kr[: t + 1] @ qr[t, a]) * m["scale"]
            p = torch.softmax(s, 0)
            out[t, a] = (p[:, None] * val[: t + 1, a]).sum(0) * gate[t, a]
    return out.reshape(S, H * dv) @ w[pre + "o"].T


def softplus(x):
    return torch.log1p(torch.exp(x))


def xielu(z, pq):
    p, q = pq[0], pq[1]
    pos = softplus(p) * z * z + z / 2
    neg = (0.5 + softplus(q)) * (torch.exp(torch.clamp(z, max=0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ff(h, w, pre):
    return xielu(h @ w[pre + "up"].T, w[pre + "act"]) @ w[pre + "down"].T


def clamped_glu_expert(h, w, pre, limit):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, -limit, limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1)
    return y @ w[pre + "down"].T


def moe_ff(h, w, pre, mlp):
    S = h.shape[0]
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[pre + "router"].T + w[pre + "router.b"]
    out = torch.zeros_like(h)
    for t in range(S):
        val, idx = torch.topk(z[t], top)
        p = torch.softmax(val, 0)
        for k in range(top):
            e = int(idx[k])
            out[t] += p[k] * clamped_glu_expert(h[t:t + 1], w, pre + "e%d." % e,
                                                mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        sh = clamped_glu_expert(h, w, pre + "shared.", mlp["shared"]["limit"])
        out = out + torch.sigmoid(h @ w[pre + "shared.sg"].T) * sh
    return out


def layer(x, w, i, spec, cfg):
    eps = cfg["norm"]["eps"]
    pre = "l%d." % i
    h = with_input_conv(scalar_norm(x, w[pre + "norm1"], eps), w[pre + "canon1"])
    assert spec["type"] == "latent_attention"
    x = x + latent_attention(h, w, pre + "mix.", spec["mixer"], eps)
    if spec.get("mlp"):
        h = with_input_conv(scalar_norm(x, w[pre + "norm2"], eps), w[pre + "canon2"])
        if spec["mlp"]["kind"] == "dense":
            x = x + dense_ff(h, w, pre + "mlp.")
        else:
            x = x + moe_ff(h, w, pre + "mlp.", spec["mlp"])
    return x


def layer_runs(cfg):
    """The order in which layers run: (layer index, pass number or None, first of its pass)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    runs += [(i, None, False) for i in range(b, n)]
    return runs


def forward(cfg, w, tokens, trace=None):
    """tokens: list of ints -> logits [S, vocab]. ``trace`` (a list) receives the
    residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x = scalar_norm(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    x0 = x
    for i, t, first in layer_runs(cfg):
        if first:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T + w["loop.step"][t]
        x = layer(x, w, i, cfg["layers"][i], cfg)
        if trace is not None:
            trace.append(x)
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].T
