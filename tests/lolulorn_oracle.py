"""Plain whole-sequence Lolulorn in float64, one function per mechanism.

Nothing here is shared with the package: no cache, no batching, no kernels.
Each function takes one sequence ``[L, ...]`` and loops where the definition
loops. ``tensors`` maps checkpoint names to tensors.
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi)
                                     * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_pairs(x, first_pos, dims, base, factor):
    """x [L, heads, d]; neighbours (2i, 2i+1) of the first ``dims`` entries
    turn by pos * base**(-2i/dims) / factor."""
    L = x.shape[0]
    out = x.clone()
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims) / factor
        a = (first_pos + torch.arange(L, dtype=F64)) * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(i, j, window, keep_first):
    return j <= i and (i - j < window or j < keep_first)


def attention_keys(h, t, pre, m, eps):
    """Keys (normed over the whole projection, then rotated) and values of a
    layer that owns them: [L, G, dim], [L, G, vdim]."""
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    L = h.shape[0]
    k = rms(h @ t[pre + "k"].to(F64).T, eps) * t[pre + "k.norm"].to(F64)
    r = m["rot"]
    k = rotate_pairs(k.reshape(L, G, d), 0, r["dims"], r["base"],
                     r["scaling"]["factor"])
    v = (h @ t[pre + "v"].to(F64).T).reshape(L, G, dv)
    return k, v


def attention(h, t, pre, m, eps, k, v):
    """h [L, W]; k, v from ``attention_keys`` of this or of the source layer."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    L = h.shape[0]
    q = rms(h @ t[pre + "q"].to(F64).T, eps) * t[pre + "q.norm"].to(F64)
    r = m["rot"]
    q = rotate_pairs(q.reshape(L, H, d), 0, r["dims"], r["base"],
                     r["scaling"]["factor"])
    win, keep = m["mask"]["size"], m["mask"]["keep_first"]
    out = torch.zeros(L, H, dv, dtype=F64)
    for i in range(L):
        js = [j for j in range(i + 1) if visible(i, j, win, keep)]
        for hh in range(H):
            g = hh // (H // G)
            p = torch.softmax(k[js, g] @ q[i, hh] * m["scale"], 0)
            out[i, hh] = p @ v[js, g]
    return out.reshape(L, H * dv) @ t[pre + "o"].to(F64).T


def causal_conv(x, w):
    """x [L, C], w [C, taps]; the last column weighs the current token."""
    L, C = x.shape
    taps = w.shape[1]
    out = torch.zeros_like(x)
    for n in range(L):
        for j in range(taps):
            src = n - (taps - 1 - j)
            if src >= 0:
                out[n] += w[:, j] * x[src]
    return out


def delta_rule(h, t, pre, m, eps):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    L = h.shape[0]

    def branch(name):
        return silu(causal_conv(h @ t[pre + name].to(F64).T,
                                t[pre + name + ".conv"].to(F64)))

    def unit(x):
        return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)

    q = unit(branch("q").reshape(L, G, d)) * d ** -0.5
    k = unit(branch("k").reshape(L, G, d))
    v = branch("v").reshape(L, H, dv)
    beta = torch.sigmoid(h @ t[pre + "b"].to(F64).T)
    dt = torch.nn.functional.softplus(h @ t[pre + "a"].to(F64).T
                                      + t[pre + "dt_bias"].to(F64))
    decay = torch.exp(-torch.exp(t[pre + "A_log"].to(F64)) * dt)
    gate = silu(h @ t[pre + "g"].to(F64).T).reshape(L, H, dv)
    out = torch.zeros(L, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for n in range(L):
            S = decay[n, hh] * S
            u = beta[n, hh] * (v[n, hh] - S.T @ k[n, g])
            S = S + torch.outer(k[n, g], u)
            out[n, hh] = S.T @ q[n, g]
    out = rms(out, eps) * t[pre + "norm"].to(F64) * gate
    return out.reshape(L, H * dv) @ t[pre + "o"].to(F64).T


def gla(h, t, pre, m, eps):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    L = h.shape[0]
    q = (h @ t[pre + "q"].to(F64).T).reshape(L, H, d) * d ** -0.5
    k = (h @ t[pre + "k"].to(F64).T).reshape(L, H, d)
    v = (h @ t[pre + "v"].to(F64).T).reshape(L, H, dv)
    z = (h @ t[pre + "a1"].to(F64).T) @ t[pre + "a2"].to(F64).T \
        + t[pre + "a2.b"].to(F64)
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).reshape(L, H, d)
    out = torch.zeros(L, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for n in range(L):
            S = alpha[n, hh][:, None] * S + torch.outer(k[n, hh], v[n, hh])
            out[n, hh] = S.T @ q[n, hh]
    out = rms(out, eps) * t[pre + "norm"].to(F64)
    out = out.reshape(L, H * dv) * silu(h @ t[pre + "g"].to(F64).T)
    return out @ t[pre + "o"].to(F64).T


def dense_ff(h, t, pre):
    a = gelu_tanh(h @ t[pre + "gate"].to(F64).T) * (h @ t[pre + "up"].to(F64).T)
    return a @ t[pre + "down"].to(F64).T


def route(h, t, pre, r):
    """Per token: chosen experts and their weights."""
    E, top = r["experts"], r["top"]
    n_groups, keep = r["groups"]["count"], r["groups"]["keep"]
    s = torch.sigmoid(h @ t[pre + "router"].to(F64).T)
    choice = s + t[pre + "correction"].to(F64)
    size = E // n_groups
    picks = []
    for n in range(h.shape[0]):
        score = []
        for g in range(n_groups):
            members = sorted(choice[n, g * size:(g + 1) * size].tolist())
            score.append(sum(members[-2:]))
        best = sorted(range(n_groups), key=lambda g: -score[g])[:keep]
        allowed = [e for e in range(E) if e // size in best]
        chosen = sorted(allowed, key=lambda e: -choice[n, e].item())[:top]
        picks.append([(e, s[n, e]) for e in chosen])
    return picks


def moe_ff(h, t, pre, mlp):
    out = torch.zeros(h.shape[0], t[pre + "e0.down"].shape[0], dtype=F64)
    for n, chosen in enumerate(route(h, t, pre, mlp["router"])):
        for e, w in chosen:
            p = f"{pre}e{e}."
            a = silu(t[p + "gate"].to(F64) @ h[n]) * (t[p + "up"].to(F64) @ h[n])
            out[n] += w * (t[p + "down"].to(F64) @ a)
    return out


def forward(cfg, t, tokens, taps=None):
    """Logits [L, vocab] of one whole sequence; ``taps`` receives the stream
    after every layer."""
    eps = cfg["norm"]["eps"]
    x = t["embed"].to(F64)[torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    kv = {}
    for i, spec in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", spec["mixer"]
        if spec["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = attention_keys(x, t, pre, m, eps)
                src = i
            y = attention(x, t, pre, m, eps, *kv[src])
        elif spec["type"] == "delta":
            y = delta_rule(x, t, pre, m, eps)
        elif spec["type"] == "gla":
            y = gla(x, t, pre, m, eps)
        else:
            raise ValueError(spec["type"])
        x = x + layer_norm(y, t[f"l{i}.norm1"].to(F64),
                           t[f"l{i}.norm1.b"].to(F64), eps)
        mlp = spec.get("mlp")
        if mlp:
            y = dense_ff(x, t, f"l{i}.mlp.") if mlp["kind"] == "dense" \
                else moe_ff(x, t, f"l{i}.mlp.", mlp)
            x = x + layer_norm(y, t[f"l{i}.norm2"].to(F64),
                               t[f"l{i}.norm2.b"].to(F64), eps)
        if taps is not None:
            taps.append(x.clone())
    x = layer_norm(x, t["final.norm"].to(F64), t["final.norm.b"].to(F64), eps)
    return x @ t["head"].to(F64).T
