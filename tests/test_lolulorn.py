"""Lolulorn through the serving path (registry -> ContinuousBatcher ->
PagedStateCache -> ops) against the plain oracle in lolulorn_oracle.py.

Every test makes its own small configuration and random tensors under the
checkpoint's names; the same tensors feed the oracle (float64) and
``load_named_tensors``. The device is the GPU when there is one (tests marked
``gpu`` then run the HIP kernels), the CPU otherwise.
"""

import json
import os

import pytest
import torch

from tests import lolulorn_oracle as O
from deepspeed_amd.inference.ragged import ContinuousBatcher, Request
from deepspeed_amd.inference.state_cache import PagedStateCache
from deepspeed_amd.models import build_model, load_pretrained

DEV = "cuda" if torch.cuda.is_available() else "cpu"


# ------------------------------------------------------------ fixtures
def att(heads=4, kv=2, dim=8, vdim=6, win=9, keep=2, dims=4, base=100.0,
        factor=1.5, kv_from=None, scale=0.45):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
         "scale": scale, "mask": {"size": win, "keep_first": keep},
         "rot": {"base": base, "dims": dims, "scaling": {"factor": factor}}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return ("attention", m)


def delta(heads=4, kv=2, dim=6, vdim=5, conv=3):
    return ("delta", {"heads": heads, "kv_heads": kv, "dim": dim,
                      "vdim": vdim, "conv": conv})


def gla(heads=2, dim=6, vdim=8, tau=8.0, rank=3):
    return ("gla", {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau,
                    "rank": rank})


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=10, groups=3, keep=2):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top,
                       "groups": {"count": groups, "keep": keep}}}


def config(layers, width=24, vocab=41, eps=1e-5, scale=3.0):
    return {"architecture": "Lolulorn", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": [{"type": kind, "mixer": m, "mlp": f}
                       for (kind, m), f in layers]}


BASE = config([(gla(), dense()), (att(), moe()), (att(kv_from=1), None),
               (delta(), moe(top=3)), (att(heads=2, kv=1, dim=6, vdim=7,
                                           win=5, keep=0, dims=6), dense(9))])


def tensors(cfg, seed=0):
    """Random tensors under the checkpoint's names, exactly representable in
    bfloat16 so both number formats start from the same weights."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def r(*shape, s=1.0):
        return (s * torch.randn(shape, generator=g)).bfloat16().float()

    def lin(o, i, s=1.5):
        return r(o, i, s=s * i ** -0.5)

    t = {"embed": r(V, W, s=0.5), "head": lin(V, W),
         "final.norm": r(W, s=0.2) + 1, "final.norm.b": r(W, s=0.2)}
    for i, spec in enumerate(cfg["layers"]):
        p, m, kind = "l%d." % i, spec["mixer"], spec["type"]
        x = p + "mix."
        for n in ("norm1", "norm2") if spec["mlp"] else ("norm1",):
            t[p + n] = r(W, s=0.2) + 1
            t[p + n + ".b"] = r(W, s=0.2)
        if kind == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[x + "q"] = lin(H * d, W)
            t[x + "q.norm"] = r(H * d, s=0.3) + 1
            if m.get("kv_from") is None:
                t[x + "k"] = lin(G * d, W)
                t[x + "v"] = lin(G * dv, W)
                t[x + "k.norm"] = r(G * d, s=0.3) + 1
            t[x + "o"] = lin(W, H * dv)
        elif kind == "delta":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
                t[x + n] = lin(rows, W)
                t[x + n + ".conv"] = r(rows, m["conv"], s=0.6)
            t[x + "b"] = lin(H, W)
            t[x + "a"] = lin(H, W)
            t[x + "A_log"] = r(H) - 1.0
            t[x + "dt_bias"] = r(H) - 1.0
            t[x + "norm"] = r(dv, s=0.2) + 1
            t[x + "g"] = lin(H * dv, W)
            t[x + "o"] = lin(W, H * dv)
        else:
            H, d, dv, rank = m["heads"], m["dim"], m["vdim"], m["rank"]
            t[x + "q"] = lin(H * d, W)
            t[x + "k"] = lin(H * d, W)
            t[x + "v"] = lin(H * dv, W)
            t[x + "g"] = lin(H * dv, W)
            t[x + "a1"] = lin(rank, W)
            t[x + "a2"] = lin(H * d, rank)
            t[x + "a2.b"] = r(H * d) + 1.0
            t[x + "norm"] = r(dv, s=0.2) + 1
            t[x + "o"] = lin(W, H * dv)
        f = spec["mlp"]
        if not f:
            continue
        if f["kind"] == "dense":
            t[p + "mlp.gate"] = lin(f["ff"], W)
            t[p + "mlp.up"] = lin(f["ff"], W)
            t[p + "mlp.down"] = lin(W, f["ff"])
        else:
            ff, E = f["expert"]["ff"], f["router"]["experts"]
            for e in range(E):
                t[p + "mlp.e%d.gate" % e] = lin(ff, W)
                t[p + "mlp.e%d.up" % e] = lin(ff, W)
                t[p + "mlp.e%d.down" % e] = lin(W, ff)
            t[p + "mlp.router"] = lin(E, W, s=3.0)
            t[p + "mlp.correction"] = r(E, s=0.5)
    return {k: v.bfloat16().float() for k, v in t.items()}


class Served:
    """A configuration loaded into the framework plus its oracle weights."""

    def __init__(self, cfg, seed=0, dtype=torch.float32, slots=4,
                 max_tokens=512, block=16, t=None):
        self.cfg = cfg
        self.t = t or tensors(cfg, seed)
        self.w64 = {k: v.double() for k, v in self.t.items()}
        self.model = build_model(cfg, dtype, self.t) \
            .load_named_tensors(self.t).to(DEV).eval()
        self.model.build_cache = self._cache(self.model.build_cache, block)
        self.batcher = ContinuousBatcher(self.model, max_slots=slots,
                                         dtype=dtype, device=torch.device(DEV),
                                         max_tokens=max_tokens)
        self.n = 0

    @staticmethod
    def _cache(build, block):
        return lambda *a, **k: build(*a, **{**k, "block_size": block})

    def oracle(self, tokens, taps=None):
        return O.forward(self.cfg, self.w64, list(tokens), taps)

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


# ------------------------------------------------- mechanisms, one by one
def test_post_norm_adds_the_normed_output_to_the_stream():
    from deepspeed_amd.ops.norms import layer_norm_add_, layer_norm_rows
    torch.manual_seed(0)
    x, y = torch.randn(5, 12) * 2, torch.randn(5, 12) * 7 + 3
    w, b = torch.randn(12), torch.randn(12)
    want = x.double() + O.layer_norm(y.double(), w.double(), b.double(), 1e-3)
    xs = x.clone().to(DEV)
    h = layer_norm_add_(xs, y.to(DEV), w.to(DEV), b.to(DEV), 1e-3,
                        torch.bfloat16)
    close(xs.cpu().double(), want, 1e-5)
    assert h.dtype == torch.bfloat16
    close(h.float().cpu().double(), want, 1e-2)
    idx = torch.tensor([3, 0])
    got = layer_norm_rows(y.to(DEV), w.to(DEV), b.to(DEV), 1e-3,
                          torch.float32, idx.to(DEV))
    close(got.cpu().double(),
          O.layer_norm(y[idx].double(), w.double(), b.double(), 1e-3), 1e-5)


def test_rotation_with_scaled_positions():
    from deepspeed_amd.ops.rope import rope_interleaved_, rope_tables
    torch.manual_seed(0)
    x = torch.randn(4, 3, 10)
    pos = torch.tensor([0, 5, 33, 60])
    cos, sin = rope_tables(6, 64, 70.0, scaling=2.5)
    got = rope_interleaved_(x.clone(), pos, cos, sin, 6)
    for i, p in enumerate(pos.tolist()):
        want = O.rotate_pairs(x[i:i + 1].double(), p, 6, 70.0, 2.5)[0]
        close(got[i].double(), want, 1e-5)
    assert torch.equal(got[..., 6:], x[..., 6:])


def test_gated_activations():
    from deepspeed_amd.ops.activations import glu
    z = torch.linspace(-6, 6, 64).reshape(2, 32)
    g, u = z[:, :16].double(), z[:, 16:].double()
    close(glu(z.to(DEV), "gelu_tanh").cpu().double(), O.gelu_tanh(g) * u, 1e-5)
    close(glu(z.to(DEV), "silu").cpu().double(), O.silu(g) * u, 1e-5)


@pytest.mark.parametrize("experts,top,groups,keep", [
    (6, 2, 3, 2), (6, 3, 3, 2), (8, 1, 4, 1), (5, 5, 1, 1), (6, 4, 2, 2),
    (4, 2, 4, 3)])
def test_router_choice_and_weights(experts, top, groups, keep):
    from deepspeed_amd.moe.routed import grouped_sigmoid_topk
    torch.manual_seed(experts * 10 + top)
    T, W = 40, 12
    h = torch.randn(T, W)
    t = {"router": torch.randn(experts, W) * 0.8,
         "correction": torch.randn(experts) * 0.7 - 0.5}   # choices go negative
    spec = {"experts": experts, "top": top,
            "groups": {"count": groups, "keep": keep}}
    want = O.route(h.double(), {k: v.double() for k, v in t.items()}, "", spec)
    logits = (h.double() @ t["router"].double().T).float()
    idx, w = grouped_sigmoid_topk(logits.to(DEV), t["correction"].to(DEV),
                                  top, groups, keep)
    for n in range(T):
        got = dict(zip(idx[n].tolist(), w[n].tolist()))
        assert sorted(got) == sorted(e for e, _ in want[n])
        for e, s in want[n]:
            assert abs(got[e] - s.item()) < 1e-5


def test_disallowed_groups_lose_even_against_negative_choices():
    from deepspeed_amd.moe.routed import grouped_sigmoid_topk
    # group 0 = {0, 1}: one high score, one very low; group 1 = {2, 3}: two
    # middling; group 2 = {4, 5}: negative choices. keep 2 of 3 groups, top 4.
    z = torch.tensor([[4.0, -9.0, 1.0, 1.0, -1.0, -1.0]])
    corr = torch.tensor([0.0, -3.0, 0.0, 0.0, -2.0, -2.0])
    idx, w = grouped_sigmoid_topk(z.to(DEV), corr.to(DEV), 4, 3, 2)
    assert sorted(idx[0].tolist()) == [0, 1, 2, 3]     # 1 is at -3, 4/5 at -1.7
    got = dict(zip(idx[0].tolist(), w[0].tolist()))
    assert abs(got[1] - torch.sigmoid(torch.tensor(-9.0)).item()) < 1e-6


@pytest.mark.parametrize("grouped", [False, True])
def test_routed_experts_match_oracle(grouped):
    cfg = config([(gla(), moe(6, 3, groups=3, keep=2))])
    s = Served(cfg)
    layer = s.model.layers[0].mlp
    if grouped:                      # the path of large steps: tokens by expert
        layer.DENSE_MAX_PICKS = 0
    torch.manual_seed(3)
    h = torch.randn(11, cfg["width"])
    want = O.moe_ff(h.double(), s.w64, "l0.mlp.", cfg["layers"][0]["mlp"])
    close(layer(h.to(DEV)).cpu().double(), want, 1e-4)


# ----------------------------------- attention reach: crafted rows and queries
def _crafted_attention(held, count, target, win, keep, G=2, rep=2, dim=4,
                       vdim=3, bs=8):
    """Rows 0..held+count-1 of one sequence; only row ``target`` has a key
    (score 40 against 0 for every head). Returns (out [count, H, vdim],
    values [L, G, vdim])."""
    from deepspeed_amd.ops.window_attention import window_attention
    g = torch.Generator().manual_seed(target + 7 * held)
    L = held + count
    cache, b = one_step_cache([G * (dim + vdim)], {}, [held], [count],
                              block=bs, tokens=L + bs)
    vals = torch.randn(L, G, vdim, generator=g)
    keys = torch.zeros(L, G, dim)
    if 0 <= target < L:
        keys[target, :, 0] = 40.0
    rows = torch.cat([keys.reshape(L, -1), vals.reshape(L, -1)], 1)
    cache.pools[0].view(-1, rows.shape[1])[pool_index(cache, 0, range(L))] = \
        rows.to(DEV)
    q = torch.zeros(count, G * rep, dim)
    q[..., 0] = 1.0
    out = window_attention(q.to(DEV), cache.pools[0], b, G, dim, vdim, 1.0,
                           win, keep).cpu().reshape(count, G * rep, vdim)
    cache.end_step()
    return out, vals


def _check_crafted(out, vals, held, target, win, keep, rep=2):
    for i in range(out.shape[0]):
        pos = held + i
        seen = [j for j in range(pos + 1) if O.visible(pos, j, win, keep)]
        for h in range(out.shape[1]):
            v = vals[:, h // rep].double()
            want = v[target] if target in seen else v[seen].mean(0)
            close(out[i, h].double(), want, 1e-4)


WIN, KEEP = 20, 3


@pytest.mark.parametrize("target", [
    0, KEEP - 1, KEEP, 7, 8,              # kept tokens, the next one, a border
    150,                                   # far behind the window
    299 - WIN, 299 - WIN + 1,              # just outside / inside for pos 299
    297, 299])
def test_decoded_token_sees_window_and_kept_tokens_only(target):
    """A single query at position 299 over 300 rows in blocks of 8, and the
    same query one position before the target (which must not see it)."""
    out, vals = _crafted_attention(299, 1, target, WIN, KEEP)
    _check_crafted(out, vals, 299, target, WIN, KEEP)
    if target > 0:
        out, vals = _crafted_attention(target - 1, 1, target, WIN, KEEP)
        _check_crafted(out, vals, target - 1, target, WIN, KEEP)


@pytest.mark.parametrize("held,count,target", [
    (0, 40, 2), (0, 40, 3), (0, 40, 19), (0, 40, 20),     # a whole prompt
    (30, 25, 2), (30, 25, 3), (30, 25, 11), (30, 25, 34), (30, 25, 35),
    (30, 25, 54), (61, 2, 42), (61, 2, 43), (61, 2, 62)])
def test_portion_queries_each_see_their_own_window(held, count, target):
    """Every query of a portion has its own edge: the target leaves the
    window of some and stays in that of others."""
    out, vals = _crafted_attention(held, count, target, WIN, KEEP)
    _check_crafted(out, vals, held, target, WIN, KEEP)


def test_no_window_and_window_wider_than_the_sequence():
    for win, keep in ((0, 0), (500, 0), (500, 4)):
        out, vals = _crafted_attention(90, 3, 1, win, keep)
        _check_crafted(out, vals, 90, 1, win if win else 10 ** 6, keep)


def test_attention_layer_matches_oracle():
    cfg = config([(att(heads=6, kv=3, dim=8, vdim=5, win=6, keep=2, dims=6),
                   None)])
    s = Served(cfg)
    t = toks(25)
    close(s.run(t, [25]), s.oracle(t))
    close(s.run(t, [3, 1, 9, 2, 1, 1, 8]), s.oracle(t))


# ------------------------------------------------- recurrences, crafted
def test_delta_rule_overwrites_a_key_and_decays():
    """One head, unit keys: writing twice under the same key replaces the
    value by beta; a decay of one half halves what is read later."""
    from deepspeed_amd.ops.linear_recurrence import linear_scan
    cache, b = one_step_cache([], {"rec": ((1, 2, 2), torch.float32)}, [0],
                              [3])
    e0 = torch.tensor([1.0, 0.0])
    q = torch.stack([e0, e0, e0]).view(3, 1, 2).to(DEV)
    k = q.clone()
    v = torch.tensor([[2.0, 4.0], [10.0, 20.0], [0.0, 0.0]]).view(3, 1, 2)
    decay = torch.tensor([[1.0], [1.0], [0.5]]).to(DEV)
    beta = torch.tensor([[1.0], [0.5], [0.0]]).to(DEV)
    o = linear_scan(q, k, v.to(DEV), decay, beta, cache.states["rec"], b)
    want = torch.tensor([[2.0, 4.0], [6.0, 12.0], [3.0, 6.0]])
    close(o.cpu().view(3, 2).double(), want.double(), 1e-6)
    close(cache.states["rec"][0, 0].cpu().double(),
          torch.tensor([[3.0, 6.0], [0.0, 0.0]]).double(), 1e-6)


def test_channel_decay_acts_on_key_rows():
    from deepspeed_amd.ops.linear_recurrence import linear_scan
    cache, b = one_step_cache([], {"rec": ((1, 2, 1), torch.float32)}, [0],
                              [2])
    k = torch.tensor([[1.0, 1.0], [0.0, 0.0]]).view(2, 1, 2).to(DEV)
    q = torch.tensor([[0.0, 0.0], [1.0, 2.0]]).view(2, 1, 2).to(DEV)
    v = torch.tensor([[3.0], [0.0]]).view(2, 1, 1).to(DEV)
    decay = torch.tensor([[1.0, 1.0], [0.5, 0.25]]).view(2, 1, 2).to(DEV)
    o = linear_scan(q, k, v, decay, None, cache.states["rec"], b,
                    q_scale=2.0)
    assert abs(o[1, 0, 0].item() - 2.0 * (1.5 + 2 * 0.75)) < 1e-6


@pytest.mark.parametrize("kind", ["delta", "gla"])
def test_recurrent_layer_matches_oracle_over_cuts(kind):
    mix = delta(heads=6, kv=2, dim=5, vdim=7, conv=4) if kind == "delta" \
        else gla(heads=3, dim=7, vdim=5, tau=3.0, rank=2)
    s = Served(config([(mix, None)]))
    t = toks(30, seed=5)
    want = s.oracle(t)
    for cuts in ([30], [1] * 30, [2, 2, 1, 13, 3, 9], [17, 13]):
        close(s.run(t, cuts), want)


def test_short_convolution_tail_is_carried_and_zero_at_the_start():
    from deepspeed_amd.ops.causal_conv import conv_silu_ragged
    torch.manual_seed(0)
    C, taps, S = 5, 4, 11
    x, w = torch.randn(S, C), torch.randn(C, taps)
    want = O.silu(O.causal_conv(x.double(), w.double()))
    for cuts in ([11], [1] * 11, [2, 1, 6, 2]):
        cache = PagedStateCache([], {"conv": (taps - 1, C)}, 2, 64,
                                block_size=8, device="cpu")
        cache.reset_slot(1)
        got, at = [], 0
        for c in cuts:
            b = cache.begin_ragged([1], [c])
            got.append(conv_silu_ragged(x[at:at + c], w,
                                        cache.states["conv"], b))
            cache.end_step()
            at += c
        close(torch.cat(got).double(), want, 1e-5)


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
    r = b.open("taps")
    got = []
    b.cache.begin_ragged([r.slot], [len(t)])
    base.model(torch.tensor(t).to(DEV), kv_cache=b.cache, taps=got)
    b.cache.end_step()
    b.close(r)
    assert len(got) == len(want)
    for x, y in zip(got, want):
        close(x.cpu().double(), y, 1e-4)


def test_unequal_batch_equals_each_alone(base):
    seqs = [toks(n, seed=10 + n) for n in (1, 7, 19, 33)]
    alone = [base.run(t, [len(t)]) for t in seqs]
    b = base.batcher
    reqs = [b.open("m%d" % i) for i in range(4)]
    first = [1, 6, 4, 17]
    out1 = b.feed([(r, t[:c]) for r, t, c in zip(reqs, seqs, first)]).cpu()
    rest = [(r, t[c:]) for r, t, c in zip(reqs, seqs, first) if len(t) > c]
    out2 = b.feed(rest).cpu()
    for r in reqs:
        b.close(r)
    at1 = at2 = 0
    for t, c, ref in zip(seqs, first, alone):
        got = [out1[at1:at1 + c]]
        at1 += c
        if len(t) > c:
            got.append(out2[at2:at2 + len(t) - c])
            at2 += len(t) - c
        close(torch.cat(got).double(), ref, 1e-4)


def test_a_request_left_out_of_steps_goes_on_later(base):
    a, c = toks(18, seed=21), toks(12, seed=22)
    b = base.batcher
    ra, rc = b.open("a"), b.open("c")
    got = [b.feed([(ra, a[:5]), (rc, c[:4])]).cpu()[:5]]
    b.feed([(rc, c[4:9])])                      # a sits this one out
    got.append(b.feed([(ra, a[5:6]), (rc, c[9:])]).cpu()[:1])
    b.close(rc)
    got.append(b.feed([(ra, a[6:])]).cpu())
    b.close(ra)
    close(torch.cat(got).double(), base.oracle(a))


def test_blocks_and_slots_are_used_again():
    """A pool of 4 blocks of 16 and 2 slots serves 6 requests in turn, each
    leaving rows, matrix states and convolution tails behind for the next."""
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
    close(base.run(t, [5] + [1] * 115), base.oracle(t))


VARIANTS = {
    # sizes that the base makes equal or 1 are unequal or larger here
    "attention_only_mha": config([(att(heads=3, kv=3, dim=6, vdim=9, win=4,
                                       keep=1, dims=2, factor=1.0), dense(7))],
                                 width=16, scale=1.0),
    "mqa_full_rotation_shared_twice": config(
        [(att(heads=5, kv=1, dim=4, vdim=4, win=7, keep=3, dims=4), None),
         (gla(heads=1, dim=9, vdim=3, tau=1.0, rank=5), moe(4, 2, 7, 4, 3)),
         (att(heads=5, kv=1, dim=4, vdim=4, win=3, keep=0, dims=4, kv_from=0),
          dense(11)),
         (att(heads=5, kv=1, dim=4, vdim=4, win=30, keep=5, dims=4,
              kv_from=0), None)], width=20, vocab=29),
    "delta_first_single_tap": config(
        [(delta(heads=2, kv=2, dim=8, vdim=3, conv=1), moe(5, 5, 6, 1, 1)),
         (delta(heads=3, kv=1, dim=4, vdim=10, conv=2), None),
         (gla(heads=4, dim=3, vdim=5, tau=20.0, rank=1), dense(13))],
        width=12, eps=1e-3, scale=7.0),
    "recurrent_then_two_caches": config(
        [(gla(heads=2, dim=5, vdim=5), None),
         (att(heads=2, kv=2, dim=10, vdim=3, win=8, keep=2, dims=6), moe()),
         (att(heads=4, kv=2, dim=6, vdim=8, win=2, keep=1, dims=2), moe(8, 3, 5, 2, 1)),
         (att(heads=2, kv=2, dim=10, vdim=3, win=5, keep=4, dims=6,
              kv_from=1), None)], width=28, vocab=53),
}


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes_and_orders(name):
    cfg = VARIANTS[name]
    s = Served(cfg, seed=3)
    t = toks(23, vocab=cfg["vocab"], seed=4)
    want = s.oracle(t)
    close(s.run(t, [23]), want)
    close(s.run(t, [4, 1, 1, 11, 2, 4]), want)


# every expert chosen: 16-bit rounding cannot flip a routing decision
SMOOTH = config([(gla(), dense()), (att(), moe(4, 4, groups=1, keep=1)),
                 (att(kv_from=1), None), (delta(), moe(4, 4, groups=2, keep=2))])


def test_bfloat16_stays_near_the_oracle():
    s = Served(SMOOTH, dtype=torch.bfloat16)
    t = toks(30, seed=6)
    want = s.oracle(t)
    close_rms(s.run(t, [30]), want, 0.08)
    close_rms(s.run(t, [7, 1, 20, 1, 1]), want, 0.08)


def test_recurrent_state_stays_32_bit_in_16_bit_serving():
    s = Served(SMOOTH, dtype=torch.bfloat16)
    st = s.batcher.cache.states
    assert st["rec0"].dtype == st["rec3"].dtype == torch.float32
    assert st["conv3"].dtype == torch.bfloat16
    assert s.batcher.cache.pools[0].dtype == torch.bfloat16
    assert len(s.batcher.cache.pools) == 1          # the borrowed rows are shared


# ---------------------------------------------- mid size, default 64-token blocks
def _mid_config(top):
    a = att(heads=8, kv=2, dim=24, vdim=20, win=40, keep=4, dims=10,
            base=3000.0, factor=2.0, scale=0.2)
    return config([(gla(heads=3, dim=20, vdim=24, tau=12.0, rank=6),
                    dense(150)),
                   (a, moe(8, top, ff=28, groups=4, keep=top // 2 or 1)),
                   (att(heads=8, kv=2, dim=24, vdim=20, win=70, keep=0,
                        dims=10, base=3000.0, factor=2.0, scale=0.2,
                        kv_from=1), None),
                   (delta(heads=6, kv=3, dim=12, vdim=18, conv=4),
                    moe(8, top, ff=36, groups=4, keep=top // 2 or 1))],
                  width=96, vocab=131, eps=1e-6, scale=5.0)


def _mixed_schedule(dtype):
    """Three requests of 150, 70 and 5 tokens share steps: portions that end
    inside, on and one past a block border beside single tokens; the short
    one ends early and its slot serves a fourth request."""
    cfg = _mid_config(2 if dtype == torch.float32 else 8)
    s = Served(cfg, seed=5, dtype=dtype, slots=3, max_tokens=64 * 6, block=64)
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
    cfg = json.loads(json.dumps(cfg))
    for spec in cfg["layers"]:
        spec["mixer"].pop("rank", None)     # a size only the tensors give
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in t.items()},
              str(folder / "model.safetensors"))


def test_registry_loads_a_checkpoint_folder(tmp_path):
    cfg = VARIANTS["delta_first_single_tap"]
    t = tensors(cfg, seed=8)
    _save(tmp_path, cfg, t)
    model = load_pretrained(str(tmp_path), dtype=torch.float32, device=DEV)
    assert model.architecture == "Lolulorn"
    b = ContinuousBatcher(model, max_slots=1, dtype=torch.float32,
                          device=torch.device(DEV), max_tokens=64)
    r = b.open("x")
    seq = toks(10, vocab=cfg["vocab"])
    got = b.feed([(r, seq)], rows=[9]).cpu().double()
    want = O.forward(cfg, {k: v.double() for k, v in t.items()}, seq)[9:]
    close(got, want)


def test_config_rejects_what_the_design_does_not_have():
    bad = config([(att(), None), (att(kv_from=1), None)])
    with pytest.raises(ValueError):
        build_model(bad)
    bad = config([(att(), None), (att(kv_from=0, dim=6), None)])
    with pytest.raises(ValueError):
        build_model(bad)
    bad = config([(gla(), None)])
    bad["layers"][0]["type"] = "conv"
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
    la, lb, lc = (O.forward(cfg, w, s) for s in (a, b, c))
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
    cfg = VARIANTS["recurrent_then_two_caches"]
    t = tensors(cfg, seed=14)
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
            seq.append(int(O.forward(cfg, w, seq)[-1].argmax()))
        assert line["generated"] == seq[len(prompt):]


# ------------------------------------------- HIP kernels against eager ops
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_match_eager_on_the_same_device(dtype, monkeypatch):
    """Same model, same schedule: HIP kernels vs the torch formulations."""
    t = toks(70, seed=12)
    cuts = [33, 1, 1, 30, 5]
    cfg = BASE if dtype == torch.float32 else SMOOTH
    k = Served(cfg, dtype=dtype)
    assert k.model.embed.is_cuda
    got = k.run(t, cuts)
    monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
    e = Served(cfg, dtype=dtype)
    want = e.run(t, cuts)
    if dtype == torch.float32:
        close(got, want, 1e-4)
    else:
        close_rms(got, want, 0.05)


@pytest.mark.gpu
def test_sequence_library_is_loaded_and_the_latent_one_is_not_needed():
    from deepspeed_amd.ops import serving_kernels as sk
    assert sk.enabled()
    Served(BASE).run(toks(5), [5])
    assert sk._libs.get("rows") is not None and sk._libs.get("seq") is not None


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mid_size_mixed_schedule_on_the_kernels(dtype):
    s, seqs, got = _mixed_schedule(dtype)
    for k, t in seqs.items():
        if dtype == torch.float32:
            close(torch.cat(got[k]), s.oracle(t), 5e-4)
        else:
            close_rms(torch.cat(got[k]), s.oracle(t), 0.15)


@pytest.mark.gpu
@pytest.mark.parametrize("dim,vdim,heads,kv", [(40, 24, 2, 1), (70, 130, 4, 2),
                                               (200, 64, 2, 2), (16, 300, 1, 1)])
@pytest.mark.parametrize("form", ["delta", "channel", "plain_scalar"])
def test_scan_kernel_sizes_against_eager(dim, vdim, heads, kv, form,
                                         monkeypatch):
    """Every register tiling of the scan (key sizes up to 256, value sizes
    that end inside a block's columns) in all three forms, a step of three
    unequal sequences continuing from non-zero states."""
    from deepspeed_amd.ops import linear_recurrence as lr
    g = torch.Generator().manual_seed(dim + vdim)
    counts, T = [9, 1, 4], 14
    if form != "delta":
        kv = heads
    cache, b = one_step_cache([], {"rec": ((heads, dim, vdim), torch.float32)},
                              [5, 0, 70], counts, tokens=1024)
    s0 = torch.randn(3, heads, dim, vdim, generator=g) * 0.1
    q = torch.randn(T, kv, dim, generator=g).to(DEV)
    k = torch.nn.functional.normalize(torch.randn(T, kv, dim, generator=g),
                                      dim=-1).to(DEV)
    v = torch.randn(T, heads, vdim, generator=g).to(DEV)
    shape = (T, heads, dim) if form == "channel" else (T, heads)
    decay = (0.5 + 0.5 * torch.rand(shape, generator=g)).to(DEV)
    beta = torch.rand(T, heads, generator=g).to(DEV) if form == "delta" \
        else None
    out = {}
    for mode in ("kernel", "eager"):
        if mode == "eager":
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        st = s0.clone().to(DEV)
        out[mode] = (lr.linear_scan(q, k, v, decay, beta, st, b, 0.7).cpu(),
                     st.cpu())
    close(out["kernel"][0].double(), out["eager"][0].double(), 1e-4)
    close(out["kernel"][1].double(), out["eager"][1].double(), 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,vdim", [(20, 2, 24, 40), (3, 3, 128, 128),
                                               (16, 1, 64, 300)])
def test_attention_kernel_sizes_against_eager(dtype, heads, kv, dim, vdim,
                                              monkeypatch):
    """More query heads per key head than one pass takes, head sizes up to
    128, a step of unequal sequences (one decoding over a long history, so
    the keys are split) over a scrambled block table."""
    from deepspeed_amd.ops import window_attention as wa
    g = torch.Generator().manual_seed(heads * dim)
    for held, counts, win, keep in (([0, 900, 37], [90, 1, 30], 300, 5),
                                    ([700, 650], [1, 2], 0, 0),
                                    ([1500], [1], 1000, 7)):
        cache = PagedStateCache([kv * (dim + vdim)], {}, len(held), 4096,
                                block_size=64, dtype=dtype, device=DEV)
        perm = torch.randperm(len(cache.free_blocks), generator=g).tolist()
        cache.free_blocks = [cache.free_blocks[i] for i in perm]
        for slot, n in enumerate(held):
            cache.reset_slot(slot)
            cache.lens[slot] = n
        b = cache.begin_ragged(list(range(len(held))), counts)
        cache.pools[0].copy_(torch.randn(cache.pools[0].shape, generator=g))
        T = sum(counts)
        q = (torch.randn(T, heads, dim, generator=g) * 0.5).to(DEV, dtype)
        got = wa.window_attention(q, cache.pools[0], b, kv, dim, vdim, 0.2,
                                  win, keep).float().cpu()
        monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        want = wa.window_attention(q, cache.pools[0], b, kv, dim, vdim, 0.2,
                                   win, keep).float().cpu()
        monkeypatch.delenv("DS_AMD_SERVING_EAGER")
        cache.end_step()
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert (got - want).abs().max().item() < tol


@pytest.mark.gpu
@pytest.mark.parametrize("heads,kv,dim,vdim", [
    (8, 2, 128, 128), (6, 3, 64, 64), (5, 1, 40, 24), (4, 4, 96, 160),
    (2, 1, 256, 256), (12, 2, 20, 6)])
def test_mfma_tiles_match_the_exact_kernel(heads, kv, dim, vdim):
    """The bf16 tile kernel against the exact one in all three size classes:
    a step of unequal portions and single tokens over a scrambled block table,
    windows that cut through tiles, kept tokens in and out of the window's
    first step, no window at all, and decoding with split keys."""
    from deepspeed_amd.ops import serving_kernels as sk
    g = torch.Generator().manual_seed(heads * dim + vdim)
    bf = torch.bfloat16
    for held, counts, win, keep in (
            ([0, 900, 37, 5], [200, 1, 130, 2], 150, 5),
            ([0], [333], 40, 0), ([10, 0], [70, 300], 100, 70),
            ([700, 650], [1, 90], 0, 0), ([1500], [1], 1000, 7),
            ([300, 0], [9, 64], 33, 33)):
        cache = PagedStateCache([kv * (dim + vdim)], {}, len(held), 4096,
                                block_size=64, dtype=bf, device=DEV)
        perm = torch.randperm(len(cache.free_blocks), generator=g).tolist()
        cache.free_blocks = [cache.free_blocks[i] for i in perm]
        for slot, n in enumerate(held):
            cache.reset_slot(slot)
            cache.lens[slot] = n
        b = cache.begin_ragged(list(range(len(held))), counts)
        cache.pools[0].copy_(torch.randn(cache.pools[0].shape, generator=g))
        T = sum(counts)
        q = (torch.randn(T, heads, dim, generator=g) * 0.5).to(DEV, bf)
        out = {}
        for path in ("mfma", "exact"):
            out[path] = sk.window_attention(q, cache.pools[0], b, kv, dim,
                                            vdim, 0.2, win, keep,
                                            path=path).float().cpu()
        cache.end_step()
        assert (out["mfma"] - out["exact"]).abs().max().item() < 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,vdim,dims", [(8, 2, 128, 128, 64),
                                                     (3, 1, 40, 24, 40),
                                                     (16, 4, 64, 8, 2),
                                                     (2, 2, 12, 20, 6)])
def test_attention_prologue_kernels_against_eager(dtype, heads, kv, dim, vdim,
                                                  dims, monkeypatch):
    """Vector path (sizes in multiples of 8) and scalar path of the prologue:
    queries, the rows written into a scrambled pool, and a borrowing layer
    that writes nothing."""
    from deepspeed_amd.ops import window_attention as wa
    from deepspeed_amd.ops.rope import rope_tables
    g = torch.Generator().manual_seed(dim)
    counts, held = [5, 1, 11], [0, 70, 9]
    T = sum(counts)
    cos, sin = rope_tables(dims, 256, 1000.0, device=DEV, scaling=2.0)
    wq = (1 + 0.3 * torch.randn(heads * dim, generator=g)).to(DEV)
    wk = (1 + 0.3 * torch.randn(kv * dim, generator=g)).to(DEV)
    for own in (True, False):
        n = heads * dim + (kv * (dim + vdim) if own else 0)
        proj = torch.randn(T, n, generator=g).to(DEV, dtype)
        res = {}
        for mode in ("kernel", "eager"):
            if mode == "eager":
                monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
            cache = PagedStateCache([kv * (dim + vdim)], {}, 3, 256,
                                    block_size=16, dtype=dtype, device=DEV)
            cache.free_blocks = cache.free_blocks[::2] + cache.free_blocks[1::2]
            for slot, m in enumerate(held):
                cache.reset_slot(slot)
                cache.lens[slot] = m
            b = cache.begin_ragged([0, 1, 2], counts)
            q = wa.attn_prep(proj, b, cache.pools[0], wq, wk, 1e-5, heads, kv,
                             dim, vdim, dims, cos, sin, own)
            res[mode] = (q.float().cpu(), cache.pools[0].float().cpu())
            cache.end_step()
        monkeypatch.delenv("DS_AMD_SERVING_EAGER")
        tol = 1e-5 if dtype == torch.float32 else 4e-2
        assert (res["kernel"][0] - res["eager"][0]).abs().max().item() < tol
        assert (res["kernel"][1] - res["eager"][1]).abs().max().item() < tol
        if not own:
            assert res["kernel"][1].abs().max().item() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff", [64, 36])
def test_gated_activation_kernels_against_eager(dtype, ff, monkeypatch):
    from deepspeed_amd.ops.activations import glu
    g = torch.Generator().manual_seed(ff)
    gu = (torch.randn(37, 2 * ff, generator=g) * 3).to(DEV, dtype)
    for act in ("silu", "gelu_tanh"):
        got = glu(gu, act).float().cpu()
        monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        want = glu(gu, act).float().cpu()
        monkeypatch.delenv("DS_AMD_SERVING_EAGER")
        tol = 1e-5 if dtype == torch.float32 else 0.1
        assert (got - want).abs().max().item() < tol * (1 + want.abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,dim,vdim,taps", [(4, 2, 128, 256, 4),
                                                     (2, 1, 16, 8, 2),
                                                     (3, 3, 24, 40, 3),
                                                     (2, 2, 10, 12, 4)])
def test_delta_prologue_kernels_against_eager(dtype, heads, kv, dim, vdim,
                                              taps, monkeypatch):
    """Vector path (multiples of 8, 2 or 4 taps) and scalar path: a step of
    unequal portions continuing from carried tails, then a second step of
    single tokens that shifts the tails."""
    from deepspeed_amd.ops import linear_recurrence as lr
    g = torch.Generator().manual_seed(dim + taps)
    C = 2 * kv * dim + heads * vdim
    n = C + heads * vdim + 2 * heads
    w = (torch.randn(C, taps, generator=g) * 0.5).to(DEV, dtype)
    a_log = (torch.randn(heads, generator=g) - 1).to(DEV)
    dtb = (torch.randn(heads, generator=g) - 1).to(DEV)
    steps = [[6, 1, 2], [1, 1, 1]]
    projs = [torch.randn(sum(c), n, generator=g).to(DEV, dtype) for c in steps]
    res = {}
    for mode in ("kernel", "eager"):
        if mode == "eager":
            monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        cache = PagedStateCache([], {"conv": (taps - 1, C)}, 3, 256,
                                block_size=16, dtype=dtype, device=DEV)
        gs = torch.Generator().manual_seed(5)
        cache.states["conv"].copy_(torch.randn(cache.states["conv"].shape,
                                               generator=gs))
        for slot, m in enumerate([9, 30, 2]):
            cache.lens[slot] = m
            if m < taps - 1:         # before a sequence's start the tail is zero
                cache.states["conv"][slot, :taps - 1 - m] = 0
        outs = []
        for counts, proj in zip(steps, projs):
            b = cache.begin_ragged([0, 1, 2], counts)
            outs += [o.float().cpu() for o in lr.delta_prep(
                proj, b, w, cache.states["conv"], a_log, dtb, kv, heads, dim,
                vdim)]
            cache.end_step()
        res[mode] = outs + [cache.states["conv"].float().cpu()]
    monkeypatch.delenv("DS_AMD_SERVING_EAGER")
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for a, b in zip(res["kernel"], res["eager"]):
        assert (a - b).abs().max().item() < tol


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
