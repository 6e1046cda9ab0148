"""Fizesun through the serving path (registry -> ContinuousBatcher ->
PagedStateCache -> ops) against the plain oracle in fizesun_oracle.py.

Every test makes its own small configuration and random tensors under the
checkpoint's names; the same tensors feed the oracle (float64) and
``load_named_tensors``. The device is the GPU when there is one (tests marked
``gpu`` then run the HIP kernels), the CPU otherwise.
"""

import json
import os

import pytest
import torch

from tests import fizesun_oracle as O
from deepspeed_amd.inference.ragged import ContinuousBatcher, Request
from deepspeed_amd.inference.state_cache import PagedStateCache
from deepspeed_amd.models import build_model, load_pretrained

DEV = "cuda" if torch.cuda.is_available() else "cpu"


# ------------------------------------------------------------ fixtures
def mixer(heads=3, dim=8, rot_dim=4, vdim=6, rank=10, dims=None, base=50.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
            "kv_rank": rank, "rot": {"base": base, "dims": dims or rot_dim},
            "scale": 0.37}


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=12, limit=1.5, shared=True):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": 8, "limit": 0.75}
    return m


def config(layers, width=24, vocab=41, taps=3, loop=None, eps=1e-5):
    cfg = {"architecture": "Fizesun", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "canon": {"taps": taps},
           "layers": [{"type": "latent_attention", "mixer": m, "mlp": f}
                      for m, f in layers]}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


BASE = config([(mixer(), dense()), (mixer(heads=2, dim=6, rank=7, dims=2),
                                    moe())], loop=(1, 2, 2))


def tensors(cfg, seed=0):
    """Random tensors under the checkpoint's names, exactly representable in
    bfloat16 so both number formats start from the same weights."""
    g = torch.Generator().manual_seed(seed)
    W, V, taps = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]

    def r(*shape, s=1.0):
        return (s * torch.randn(shape, generator=g)).bfloat16().float()

    def lin(o, i):
        return r(o, i, s=1.5 * i ** -0.5)

    t = {"embed": r(V, W), "embed.norm": r(s=0.2) + 1, "head": lin(V, W),
         "final.norm": r(s=0.2) + 1}
    if cfg.get("loop"):
        t["loop.in"] = lin(W, 2 * W)
        t["loop.step"] = r(cfg["loop"]["times"], W, s=0.3)
    for i, spec in enumerate(cfg["layers"]):
        p, m = "l%d." % i, spec["mixer"]
        H = m["heads"]
        t[p + "norm1"] = r(s=0.2) + 1
        t[p + "canon1"] = r(W, taps, s=0.4)
        t[p + "mix.q"] = lin(H * (m["dim"] + m["rot_dim"]), W)
        t[p + "mix.dkv"] = lin(m["kv_rank"] + m["rot_dim"], W)
        t[p + "mix.dkv.norm"] = r(m["kv_rank"], s=0.2) + 1
        t[p + "mix.uk"] = lin(H * m["dim"], m["kv_rank"])
        t[p + "mix.uv"] = lin(H * m["vdim"], m["kv_rank"])
        t[p + "mix.g"] = lin(H, W)
        t[p + "mix.o"] = lin(W, H * m["vdim"])
        f = spec["mlp"]
        if not f:
            continue
        t[p + "norm2"] = r(s=0.2) + 1
        t[p + "canon2"] = r(W, taps, s=0.4)
        if f["kind"] == "dense":
            t[p + "mlp.up"] = lin(f["ff"], W)
            t[p + "mlp.down"] = lin(W, f["ff"])
            t[p + "mlp.act"] = r(2, s=0.5)
        else:
            ff = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                t[p + "mlp.e%d.gate" % e] = lin(ff, W)
                t[p + "mlp.e%d.up" % e] = lin(ff, W)
                t[p + "mlp.e%d.down" % e] = lin(W, ff)
            t[p + "mlp.router"] = lin(f["router"]["experts"], W)
            t[p + "mlp.router.b"] = r(f["router"]["experts"], s=0.3)
            if f.get("shared"):
                sf = f["shared"]["ff"]
                t[p + "mlp.shared.gate"] = lin(sf, W)
                t[p + "mlp.shared.up"] = lin(sf, W)
                t[p + "mlp.shared.down"] = lin(W, sf)
                t[p + "mlp.shared.sg"] = lin(1, W)
    return {k: v.bfloat16().float() for k, v in t.items()}


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

    def oracle(self, tokens):
        return O.forward(self.cfg, self.w64, list(tokens))

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


# ------------------------------------------------- mechanisms, one by one
def test_norm_conv_matches_oracle_over_cuts():
    from deepspeed_amd.ops.causal_conv import norm_conv_ragged
    torch.manual_seed(0)
    _norm_conv_case(4)
    _norm_conv_case(9)      # longer than the filters the tiled kernel covers


def _norm_conv_case(taps):
    from deepspeed_amd.ops.causal_conv import norm_conv_ragged
    C, S = 10, 9
    x = torch.randn(S, C) * 3
    g, w = torch.tensor([1.3]), torch.randn(C, taps) * 0.5
    want = O.with_input_conv(O.scalar_norm(x.double(), g.double(), 1e-5),
                             w.double())
    for cuts in ([9], [1] * 9, [2, 5, 1, 1], [4, 2, 3]):
        cache = PagedStateCache([4], {"conv": (3, taps - 1, C)}, 2, 64,
                                block_size=8, device=DEV)
        cache.reset_slot(1)
        got, at = [], 0
        for c in cuts:
            b = cache.begin_ragged([1], [c])
            got.append(norm_conv_ragged(x[at:at + c].to(DEV).contiguous(),
                                        g.to(DEV), 1e-5, w.to(DEV),
                                        cache.states["conv"][:, 1], b,
                                        torch.float32).cpu())
            cache.end_step()
            at += c
        close(torch.cat(got).double(), want, 1e-5)


def test_single_tap_conv_and_no_state():
    s = Served(config([(mixer(), dense())], taps=1))
    t = toks(7)
    close(s.run(t, [3, 1, 3]), s.oracle(t))


def test_rotation_pairs_adjacent_dims_and_leaves_the_rest():
    from deepspeed_amd.ops.rope import rope_interleaved_, rope_tables
    torch.manual_seed(0)
    x = torch.randn(5, 2, 6)
    pos = torch.tensor([0, 3, 4, 17, 30])
    cos, sin = rope_tables(4, 64, 50.0)
    got = rope_interleaved_(x.clone(), pos, cos, sin, 4)
    for i, p in enumerate(pos.tolist()):
        want = O.rotate_pairs(x[i].double(), p, 4, 50.0)
        close(got[i].double(), want, 1e-5)
    assert torch.equal(got[..., 4:], x[..., 4:])


def test_xielu_both_branches():
    from deepspeed_amd.ops.activations import xielu
    z = torch.linspace(-6, 6, 101).reshape(1, -1)
    pq = torch.tensor([0.4, -0.7])
    close(xielu(z.to(DEV), pq.to(DEV)).cpu().double(),
          O.xielu(z.double(), pq.double()), 1e-5)


def test_clamped_expert_limits_bite():
    from deepspeed_amd.ops.activations import clamped_swiglu
    torch.manual_seed(0)
    gu = torch.randn(6, 10) * 3          # far beyond the limit on both sides
    lim = 0.8
    g = torch.clamp(gu[:, :5].double(), max=lim)
    u = torch.clamp(gu[:, 5:].double(), -lim, lim)
    want = g * torch.sigmoid(1.702 * g) * (u + 1)
    close(clamped_swiglu(gu.to(DEV), lim).cpu().double(), want, 1e-5)


@pytest.mark.parametrize("experts,top,shared", [(5, 2, True), (4, 4, False),
                                                 (3, 1, True)])
@pytest.mark.parametrize("grouped", [False, True])
def test_routed_experts_match_oracle(experts, top, shared, grouped):
    cfg = config([(mixer(), moe(experts, top, shared=shared))])
    s = Served(cfg)
    layer = s.model.layers[0].mlp
    if grouped:                      # the path of large steps: tokens by expert
        layer.DENSE_MAX_PICKS = 0
    torch.manual_seed(3)
    h = torch.randn(11, cfg["width"])
    want = O.moe_ff(h.double(), s.w64, "l0.mlp.", cfg["layers"][0]["mlp"])
    close(layer(h.to(DEV)).cpu().double(), want, 1e-4)


def test_router_weights_are_softmax_over_chosen_only():
    from deepspeed_amd.moe.routed import topk_softmax
    z = torch.tensor([[0.1, 5.0, -2.0, 4.0, 3.9]])
    idx, w = topk_softmax(z.to(DEV), 2)
    assert sorted(idx[0].tolist()) == [1, 3]
    want = torch.softmax(torch.tensor([5.0, 4.0]), 0)
    got = w[0].cpu()[torch.argsort(idx[0].cpu())]
    close(got.double(), want.double(), 1e-5)


# ----------------------------------- attention reach: crafted rows and queries
def _attend(cache, q_lat, q_rot, rank, scale=1.0):
    from deepspeed_amd.ops.latent_attention import latent_attention
    return latent_attention(q_lat.to(DEV), q_rot.to(DEV), cache.pools[0],
                            cache.batch, rank, scale).cpu()


@pytest.mark.parametrize("target", [0, 1, 7, 8, 9, 15, 16, 17, 150, 298, 299])
def test_a_far_key_is_found_and_a_future_key_is_not(target):
    """300 cached rows in blocks of 8; row ``target`` alone matches the
    query (score 40 against 0), so the output must be its latent. The same
    query one position BEFORE the target must not see it."""
    rank, rot, L, bs = 6, 2, 300, 8
    g = torch.Generator().manual_seed(target)
    cache = PagedStateCache([rank + rot], {}, 2, 320, block_size=bs,
                            device=DEV)
    lat = torch.randn(L, rank, generator=g)
    rows = torch.cat([lat, torch.zeros(L, rot)], 1)
    rows[:, rank] = 0.0
    rows[target, rank] = 40.0           # the only key with a rotated part
    q_lat = torch.zeros(1, 1, rank)
    q_rot = torch.zeros(1, 1, rot)
    q_rot[0, 0, 0] = 1.0
    for qpos, sees in ((L - 1, True), (target, True), (target - 1, False)):
        if qpos < 0:
            continue
        cache.reset_slot(0)
        cache.lens[0] = qpos             # the query is the token at qpos
        b = cache.begin_ragged([0], [1])
        tab = cache.block_table[0]
        idx = torch.tensor([tab[p // bs] * bs + p % bs
                            for p in range(qpos + 1)])
        cache.pools[0].view(-1, rank + rot)[idx.to(DEV)] = \
            rows[:qpos + 1].to(DEV)
        out = _attend(cache, q_lat, q_rot, rank)[0, 0]
        cache.end_step()
        if sees:
            close(out.double(), lat[target].double(), 1e-4)
        else:
            want = lat[:qpos + 1].mean(0)      # all scores equal
            close(out.double(), want.double(), 1e-4)


def test_portion_queries_see_exactly_their_own_past():
    """A portion of 5 queries over 20 held rows: query i sees rows 0..20+i."""
    rank, rot, bs = 4, 2, 8
    torch.manual_seed(0)
    cache = PagedStateCache([rank + rot], {}, 1, 64, block_size=bs, device=DEV)
    cache.reset_slot(0)
    cache.lens[0] = 20
    b = cache.begin_ragged([0], [5])
    rows = torch.randn(25, rank + rot)
    tab = cache.block_table[0]
    idx = torch.tensor([tab[p // bs] * bs + p % bs for p in range(25)])
    cache.pools[0].view(-1, rank + rot)[idx.to(DEV)] = rows.to(DEV)
    q_lat, q_rot = torch.randn(2, 5, rank), torch.randn(5, 2, rot)
    out = _attend(cache, q_lat, q_rot, rank, 0.5)
    for h in range(2):
        for i in range(5):
            k = rows[:21 + i].double()
            s = (k[:, :rank] @ q_lat[h, i].double()
                 + k[:, rank:] @ q_rot[i, h].double()) * 0.5
            want = torch.softmax(s, 0) @ k[:, :rank]
            close(out[h, i].double(), want, 1e-4)


# ------------------------------------------------ whole model, schedules
@pytest.fixture(scope="module")
def base():
    return Served(BASE)


def test_first_tokens(base):
    for n in (1, 2, 3):
        t = toks(n, seed=n)
        close(base.run(t, [n]), base.oracle(t))


def test_prefill_equals_token_by_token(base):
    t = toks(21)
    want = base.oracle(t)
    close(base.run(t, [21]), want)
    close(base.run(t, [1] * 21), want)


@pytest.mark.parametrize("cuts", [[2] * 18, [3, 2, 16, 1, 14], [15, 1, 17, 3],
                                  [17, 2, 1, 16], [31, 5], [16, 16, 4]])
def test_portions_cut_anywhere(base, cuts):
    t = toks(36, seed=5)                # block size 16: cuts on and off edges
    close(base.run(t, cuts), base.oracle(t))


def test_layer_streams_match_oracle(base):
    t = toks(9, seed=2)
    want = []
    O.forward(base.cfg, base.w64, t, want)
    req = base.batcher.open("streams")
    got = []
    base.batcher.cache.begin_ragged([req.slot], [len(t)])
    base.model(torch.tensor(t, device=DEV), kv_cache=base.batcher.cache,
               taps=got)
    base.batcher.cache.end_step()
    base.batcher.close(req)
    assert len(got) == len(want) == 3   # layer 0 once, layer 1 twice
    for a, b in zip(got, want):
        close(a.cpu().double(), b)


def test_unequal_batch_equals_each_alone(base):
    seqs = [toks(n, seed=10 + n) for n in (1, 7, 19, 33)]
    alone = [base.run(t, [len(t)]) for t in seqs]
    b = base.batcher
    reqs = [b.open("m%d" % i) for i in range(4)]
    # step 1: whole short ones, portions of long ones; step 2: the rest
    # beside single tokens
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


def test_blocks_and_slots_are_used_again():
    """A pool of 4 blocks of 16 and 2 slots serves 6 requests in turn, each
    leaving rows and convolution tails behind for the next owner."""
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


def test_long_decode(base):
    t = toks(120, seed=9)
    close(base.run(t, [5] + [1] * 115), base.oracle(t))


VARIANTS = {
    "no_loop": config([(mixer(), dense()), (mixer(), moe())]),
    "loop_all_once": config([(mixer(), moe(top=1)), (mixer(), dense())],
                            loop=(0, 2, 1)),
    "loop_tail_thrice": config([(mixer(), dense()), (mixer(heads=1), None)],
                               loop=(1, 2, 3), taps=2),
    "one_head_wide_rot": config([(mixer(heads=1, dim=4, rot_dim=8, vdim=9,
                                        rank=5, dims=6), dense(7))],
                                width=16, taps=5),
    "no_unrotated_state_equalities": config(
        [(mixer(heads=4, dim=5, rot_dim=2, vdim=3, rank=9), moe(6, 6, ff=5)),
         (mixer(heads=2, dim=12, rot_dim=6, vdim=8, rank=4, dims=4),
          dense(33))], width=20, vocab=29, loop=(0, 1, 2)),
}


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes_and_orders(name):
    cfg = VARIANTS[name]
    s = Served(cfg, seed=3)
    t = toks(19, vocab=cfg["vocab"], seed=4)
    want = s.oracle(t)
    close(s.run(t, [19]), want)
    close(s.run(t, [4, 1, 1, 11, 2]), want)


# every expert chosen: 16-bit rounding cannot flip a routing decision
SMOOTH = config([(mixer(), dense()), (mixer(heads=2, dim=6, rank=7, dims=2),
                                      moe(4, 4))], loop=(1, 2, 2))


def test_bfloat16_stays_near_the_oracle():
    s = Served(SMOOTH, dtype=torch.bfloat16)
    t = toks(30, seed=6)
    want = s.oracle(t)
    close_rms(s.run(t, [30]), want, 0.06)
    close_rms(s.run(t, [7, 1, 20, 1, 1]), want, 0.06)


# ---------------------------------------------- mid size, default 64-token blocks
def _mid_config(top):
    a = mixer(heads=5, dim=24, rot_dim=12, vdim=20, rank=40, dims=8, base=3000.0)
    b = mixer(heads=2, dim=32, rot_dim=8, vdim=32, rank=24, base=700.0)
    return config([(a, moe(6, top, ff=28, limit=1.2, shared=False)),
                   (b, dense(150)), (a, moe(6, top, ff=36, limit=3.0))],
                  width=96, vocab=131, taps=5, loop=(0, 2, 2), eps=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mid_size_mixed_schedule_over_block_borders(dtype):
    """Three requests of 150, 70 and 5 tokens share steps: portions that end
    on and off the 64-token block borders beside single tokens; five layer
    runs with two attention shapes."""
    cfg = _mid_config(3 if dtype == torch.float32 else 6)
    s = Served(cfg, seed=21, dtype=dtype, slots=3, max_tokens=64 * 6, block=64)
    seqs = {"a": toks(150, 131, seed=31), "b": toks(70, 131, seed=32),
            "c": toks(5, 131, seed=33)}
    steps = [{"a": 67, "b": 2}, {"a": 61, "b": 62, "c": 5}, {"a": 1, "b": 1},
             {"a": 1, "b": 1}, {"b": 4, "a": 2}, {"a": 18}]
    reqs, at, got = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in steps:
        entries = []
        for k, n in step.items():
            if k not in reqs:
                reqs[k] = s.batcher.open(k)
            entries.append((reqs[k], seqs[k][at[k]:at[k] + n]))
        out = s.batcher.feed(entries).double().cpu()
        o = 0
        for k, n in step.items():
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
            if at[k] == len(seqs[k]):
                s.batcher.close(reqs[k])
    for k, t in seqs.items():
        assert at[k] == len(t)
        if dtype == torch.float32:
            close(torch.cat(got[k]), s.oracle(t), 3e-4)
        else:
            # five layer runs of unit-gain random weights amplify 16-bit
            # rounding; the sharp comparison is the 32-bit one above
            close_rms(torch.cat(got[k]), s.oracle(t), 0.15)


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


def test_registry_loads_a_checkpoint_folder(tmp_path):
    from safetensors.torch import save_file
    cfg = VARIANTS["loop_tail_thrice"]
    t = tensors(cfg, seed=8)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in t.items()},
              str(tmp_path / "model.safetensors"))
    model = load_pretrained(str(tmp_path), dtype=torch.float32, device=DEV)
    b = ContinuousBatcher(model, max_slots=1, dtype=torch.float32,
                          device=torch.device(DEV), max_tokens=64)
    r = b.open("x")
    seq = toks(10, vocab=cfg["vocab"])
    got = b.feed([(r, seq)], rows=[9]).cpu().double()
    want = O.forward(cfg, {k: v.double() for k, v in t.items()}, seq)[9:]
    close(got, want)


def test_schedule_replay_runner(tmp_path):
    """bin/trace_run end to end: two requests, portions beside single tokens,
    a slot used again; logits files against the oracle."""
    import subprocess
    import sys
    import numpy as np
    from safetensors.torch import save_file
    cfg = BASE
    t = tensors(cfg, seed=11)
    mdir, out = tmp_path / "m", tmp_path / "o"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in t.items()},
              str(mdir / "model.safetensors"))
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
    from safetensors.torch import save_file
    cfg = VARIANTS["no_loop"]
    t = tensors(cfg, seed=14)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in t.items()},
              str(tmp_path / "model.safetensors"))
    a, b = toks(6, seed=70), toks(6, seed=71)
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
def test_serving_library_is_loaded():
    from deepspeed_amd.ops import serving_kernels as sk
    assert sk.enabled()
    Served(BASE).run(toks(5), [5])
    assert sk._libs.get("rows") is not None


@pytest.mark.gpu
def test_split_key_decode_over_long_history():
    """Few query tokens over a long history take the split-key path."""
    s = Served(config([(mixer(), dense())]), max_tokens=2048, block=64)
    t = toks(1500, seed=13)
    got = s.run(t, [1490] + [1] * 10)[-10:]
    close(got, s.oracle(t)[-10:], 5e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("heads,rank,rot", [(3, 20, 6), (7, 56, 8),
                                            (5, 96, 32), (4, 200, 40),
                                            (2, 512, 64)])
def test_mfma_tiles_match_the_exact_kernel(heads, rank, rot):
    """Ragged batch (held tokens, portions of unequal length, a single decoded
    token) over 16-token blocks handed out in scrambled order."""
    from deepspeed_amd.ops import serving_kernels as sk
    g = torch.Generator().manual_seed(rank)
    bs = 16
    cache = PagedStateCache([rank + rot], {}, 4, 2048, block_size=bs,
                            dtype=torch.bfloat16, device=DEV)
    perm = torch.randperm(cache.num_blocks, generator=g).tolist()
    cache.free_blocks = perm
    held, counts = [0, 37, 300, 129], [150, 1, 77, 200]
    for slot, n in enumerate(held):
        cache.lens[slot] = n
    b = cache.begin_ragged([0, 1, 2, 3], counts)
    cache.pools[0].copy_(torch.randn(cache.pools[0].shape, generator=g))
    T = sum(counts)
    q_lat = (torch.randn(heads, T, rank, generator=g) * 0.3).to(
        DEV, torch.bfloat16)
    q_rot = torch.randn(T, heads, rot, generator=g).to(DEV, torch.bfloat16)
    a = sk.latent_attention(q_lat, q_rot, cache.pools[0], b, rank, 0.2,
                            path="mfma").float().cpu()
    e = sk.latent_attention(q_lat, q_rot, cache.pools[0], b, rank, 0.2,
                            path="exact").float().cpu()
    # the weights are rounded to 16 bits before the second product
    assert (a - e).abs().max().item() < 0.03
    assert ((a - e) ** 2).mean().sqrt().item() < 0.004


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_exact_kernel_with_more_heads_than_one_group(dtype, monkeypatch):
    """11 heads (the exact kernel walks heads in groups of 8), with and
    without key splits, against the eager formulation."""
    from deepspeed_amd.ops import latent_attention as la
    from deepspeed_amd.ops import serving_kernels as sk
    heads, rank, rot, bs = 11, 40, 8, 16
    g = torch.Generator().manual_seed(5)
    cache = PagedStateCache([rank + rot], {}, 3, 2048, block_size=bs,
                            dtype=dtype, device=DEV)
    for held, counts in (([0, 200, 37], [90, 1, 30]), ([700, 650], [1, 2])):
        for slot in range(3):
            cache.reset_slot(slot)
        for slot, n in enumerate(held):
            cache.lens[slot] = n
        b = cache.begin_ragged(list(range(len(held))), counts)
        cache.pools[0].copy_(torch.randn(cache.pools[0].shape, generator=g))
        T = sum(counts)
        q_lat = (torch.randn(heads, T, rank, generator=g) * 0.3).to(DEV, dtype)
        q_rot = torch.randn(T, heads, rot, generator=g).to(DEV, dtype)
        got = sk.latent_attention(q_lat, q_rot, cache.pools[0], b, rank, 0.2,
                                  path="exact").float().cpu()
        monkeypatch.setenv("DS_AMD_SERVING_EAGER", "1")
        want = la.latent_attention(q_lat, q_rot, cache.pools[0], b, rank,
                                   0.2).float().cpu()
        monkeypatch.delenv("DS_AMD_SERVING_EAGER")
        cache.end_step()
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        assert (got - want).abs().max().item() < tol
