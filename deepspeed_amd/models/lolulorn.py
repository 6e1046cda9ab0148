"""Lolulorn: a decoder-only serving model whose layers mix three kinds of
sequence mixers, assembled from the framework's ragged-batch mechanisms.

* residual stream in fp32; sublayers read the stream itself and their OUTPUT
  is layer-normed (weight and bias) before it is added
  (ops/norms.py ``layer_norm_add_``);
* mixer ``attention``: grouped-query attention over paged K/V rows with an RMS
  norm over the whole query / key projection, interleaved partial rotary with
  linear position scaling, and a sliding window that keeps the first tokens
  (ops/window_attention.py); a layer may read another layer's rows
  (``kv_from``) instead of caching its own;
* mixer ``delta``: gated delta rule with short convolutions on q, k, v;
* mixer ``gla``: gated linear attention with a low-rank per-channel decay
  (both ops/linear_recurrence.py, fp32 matrix state per request slot);
* feed-forward: dense GeGLU (tanh form) or routed SiLU-gated experts chosen by
  a sigmoid router with a choice correction and group-limited top-k
  (moe/routed.py).

The model runs only through a ``PagedStateCache`` step: ``forward`` takes the
flat token list of a ragged batch. Every size and constant comes from the
config.
"""

from dataclasses import dataclass
from typing import List

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..inference.state_cache import PagedStateCache
from ..moe.routed import RoutedExperts
from ..ops.activations import glu
from ..ops.linear_recurrence import (delta_prep, head_norm_gate, linear_scan,
                                     sigmoid_pow)
from ..ops.norms import embed_rows, layer_norm_add_, layer_norm_rows
from ..ops.rope import rope_tables
from ..ops.window_attention import attn_prep, window_attention

MIXERS = ("attention", "delta", "gla")


@dataclass
class LolulornConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    max_seq_len: int = 1 << 16

    @classmethod
    def from_dict(cls, d: dict) -> "LolulornConfig":
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]),
                  layers=list(d["layers"]), norm_eps=float(d["norm"]["eps"]),
                  embed_scale=float((d.get("embedding") or {})
                                    .get("scale", 1.0)))
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": "Lolulorn", "vocab": self.vocab_size,
                "width": self.width, "layers": self.layers,
                "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embed_scale}}

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def validate(self):
        for i, spec in enumerate(self.layers):
            if spec["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {spec['type']!r}")
            src = spec["mixer"].get("kv_from")
            if src is None:
                continue
            if spec["type"] != "attention" or not 0 <= int(src) < i or \
                    self.layers[int(src)]["type"] != "attention" or \
                    self.layers[int(src)]["mixer"].get("kv_from") is not None:
                raise ValueError(f"layer {i}: kv_from must name an earlier "
                                 "attention layer with rows of its own")
            a, b = spec["mixer"], self.layers[int(src)]["mixer"]
            if any(a.get(k, a["heads"]) != b.get(k, b["heads"])
                   for k in ("kv_heads", "dim", "vdim", "rot")):
                raise ValueError(f"layer {i}: kv_from layer differs in shape")


def _w(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


class WindowAttention(nn.Module):
    """Fused input projection q | k | v (q alone when the rows are another
    layer's)."""

    def __init__(self, width, m: dict, eps, dtype):
        super().__init__()
        self.heads = int(m["heads"])
        self.kv_heads = int(m.get("kv_heads", self.heads))
        self.dim, self.vdim = int(m["dim"]), int(m.get("vdim", m["dim"]))
        rot = m.get("rot") or {}
        self.rot_dims = int(rot.get("dims", 0))
        self.rot_base = float(rot.get("base", 10000.0))
        self.rot_factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        if self.heads % self.kv_heads or self.rot_dims % 2 or \
                self.rot_dims > self.dim:
            raise ValueError("attention: heads must be a multiple of kv_heads "
                             "and rot.dims even and at most dim")
        self.scale = float(m["scale"])
        mask = m.get("mask") or {}
        self.window = int(mask.get("size", 0))
        self.keep_first = int(mask.get("keep_first", 0))
        self.kv_from = m.get("kv_from")
        self.own_kv = self.kv_from is None
        self.eps = eps
        nq = self.heads * self.dim
        nkv = self.kv_heads * (self.dim + self.vdim) if self.own_kv else 0
        self.w_in = _w(nq + nkv, width, dtype=dtype)
        self.q_norm = _w(nq, dtype=torch.float32)
        self.k_norm = _w(self.kv_heads * self.dim, dtype=torch.float32) \
            if self.own_kv else None
        self.w_o = _w(width, self.heads * self.vdim, dtype=dtype)

    @property
    def row_dim(self):
        return self.kv_heads * (self.dim + self.vdim)

    def forward(self, h, cache: PagedStateCache, stream, slot_states):
        b = cache.batch
        cos, sin = rope_tables(self.rot_dims, cache.max_seq, self.rot_base,
                               device=h.device, scaling=self.rot_factor)
        pool = cache.pools[stream]
        q = attn_prep(F.linear(h, self.w_in), b, pool, self.q_norm,
                      self.k_norm, self.eps, self.heads, self.kv_heads,
                      self.dim, self.vdim, self.rot_dims, cos, sin,
                      self.own_kv)
        o = window_attention(q, pool, b, self.kv_heads, self.dim, self.vdim,
                             self.scale, self.window, self.keep_first)
        return F.linear(o, self.w_o)


class GatedDeltaRule(nn.Module):
    """Fused input projection q | k | v | gate | b | a."""

    def __init__(self, width, m: dict, eps, dtype):
        super().__init__()
        self.heads = int(m["heads"])
        self.kv_heads = int(m.get("kv_heads", self.heads))
        self.dim, self.vdim, self.taps = int(m["dim"]), int(m["vdim"]), \
            int(m.get("conv", 1))
        if self.heads % self.kv_heads or self.taps < 1:
            raise ValueError("delta: heads must be a multiple of kv_heads")
        self.eps = eps
        nqk, nv = self.kv_heads * self.dim, self.heads * self.vdim
        self.conv_channels = 2 * nqk + nv
        self.w_in = _w(self.conv_channels + nv + 2 * self.heads, width,
                       dtype=dtype)
        self.conv = _w(self.conv_channels, self.taps, dtype=dtype)
        self.a_log = _w(self.heads, dtype=torch.float32)
        self.dt_bias = _w(self.heads, dtype=torch.float32)
        self.norm = _w(self.vdim, dtype=torch.float32)
        self.w_o = _w(width, nv, dtype=dtype)

    def state_shapes(self, dtype):
        return {"conv": ((max(self.taps - 1, 0), self.conv_channels), dtype),
                "rec": ((self.heads, self.dim, self.vdim), torch.float32)}

    def forward(self, h, cache: PagedStateCache, stream, slot_states):
        b = cache.batch
        proj = F.linear(h, self.w_in)
        q, k, v, beta, decay = delta_prep(
            proj, b, self.conv, slot_states["conv"], self.a_log, self.dt_bias,
            self.kv_heads, self.heads, self.dim, self.vdim)
        o = linear_scan(q, k, v, decay, beta, slot_states["rec"], b)
        C, nv = self.conv_channels, self.heads * self.vdim
        y = head_norm_gate(o, self.norm, proj[:, C:C + nv], self.eps, h.dtype)
        return F.linear(y, self.w_o)


class GatedLinearAttention(nn.Module):
    """Fused input projection q | k | v | gate | a1 (the low-rank decay's
    first factor); the second factor is a GEMM of its own."""

    def __init__(self, width, m: dict, eps, dtype, rank):
        super().__init__()
        self.heads, self.dim, self.vdim = int(m["heads"]), int(m["dim"]), \
            int(m["vdim"])
        self.inv_tau = 1.0 / float(m["tau"])
        self.rank, self.eps = rank, eps
        nk, nv = self.heads * self.dim, self.heads * self.vdim
        self.w_in = _w(2 * nk + 2 * nv + rank, width, dtype=dtype)
        self.w_a2 = _w(nk, rank, dtype=dtype)
        self.a2_bias = _w(nk, dtype=torch.float32)
        self.norm = _w(self.vdim, dtype=torch.float32)
        self.w_o = _w(width, nv, dtype=dtype)

    def state_shapes(self, dtype):
        return {"rec": ((self.heads, self.dim, self.vdim), torch.float32)}

    def forward(self, h, cache: PagedStateCache, stream, slot_states):
        b = cache.batch
        T, H, d, dv = h.shape[0], self.heads, self.dim, self.vdim
        nk, nv = H * d, H * dv
        proj = F.linear(h, self.w_in)
        z = F.linear(proj[:, 2 * nk + 2 * nv:], self.w_a2)
        alpha = sigmoid_pow(z, self.a2_bias, self.inv_tau).view(T, H, d)
        o = linear_scan(proj[:, :nk].view(T, H, d),
                        proj[:, nk:2 * nk].view(T, H, d),
                        proj[:, 2 * nk:2 * nk + nv].view(T, H, dv), alpha,
                        None, slot_states["rec"], b, q_scale=d ** -0.5)
        y = head_norm_gate(o, self.norm,
                           proj[:, 2 * nk + nv:2 * nk + 2 * nv], self.eps,
                           h.dtype)
        return F.linear(y, self.w_o)


class GatedMLP(nn.Module):
    """down(act(gate h) * (up h)); gate and up rows fused."""

    def __init__(self, width, ff, act, dtype):
        super().__init__()
        self.act = act
        self.w_gu = _w(2 * ff, width, dtype=dtype)
        self.w_down = _w(width, ff, dtype=dtype)

    def forward(self, h):
        return F.linear(glu(F.linear(h, self.w_gu), self.act), self.w_down)


class PostNorm(nn.Module):
    """Weight and bias of a layer norm applied to a sublayer's output."""

    def __init__(self, width, eps):
        super().__init__()
        self.weight = _w(width, dtype=torch.float32)
        self.bias = _w(width, dtype=torch.float32)
        self.eps = eps


class LolulornLayer(nn.Module):
    def __init__(self, cfg: LolulornConfig, spec: dict, dtype, a1_rank=0):
        super().__init__()
        W, eps, m = cfg.width, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "attention":
            self.mixer = WindowAttention(W, m, eps, dtype)
        elif self.kind == "delta":
            self.mixer = GatedDeltaRule(W, m, eps, dtype)
        elif self.kind == "gla":
            self.mixer = GatedLinearAttention(W, m, eps, dtype, a1_rank)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = PostNorm(W, eps)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp:
            self.norm2 = PostNorm(W, eps)
            if mlp["kind"] == "dense":
                self.mlp = GatedMLP(W, int(mlp["ff"]), "gelu_tanh", dtype)
            elif mlp["kind"] == "moe":
                r = mlp["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                self.mlp = RoutedExperts(
                    W, int(mlp["expert"]["ff"]), int(r["experts"]),
                    int(r["top"]), dtype=dtype, activation="silu",
                    router="sigmoid_grouped",
                    groups=(int(g["count"]), int(g["keep"])))
            else:
                raise ValueError(f"unknown mlp kind {mlp['kind']!r}")

    def forward(self, x, h, cache, stream, slot_states, dtype):
        """x: fp32 stream, updated in place; h: the stream in the compute
        dtype (x itself in fp32 mode). Returns the new h."""
        n1 = self.norm1
        h = layer_norm_add_(x, self.mixer(h, cache, stream, slot_states),
                            n1.weight, n1.bias, n1.eps, dtype)
        if self.mlp is not None:
            n2 = self.norm2
            h = layer_norm_add_(x, self.mlp(h), n2.weight, n2.bias, n2.eps,
                                dtype)
        return h


class LolulornForCausalLM(nn.Module):
    architecture = "Lolulorn"

    def __init__(self, cfg: LolulornConfig, dtype=torch.bfloat16,
                 a1_ranks=None):
        """``a1_ranks[i]``: rank of layer i's low-rank decay projection (a
        size the tensors give, not the config); default ``dim // 2``."""
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        W = cfg.width
        a1_ranks = a1_ranks or {}
        self.embed = _w(cfg.vocab_size, W, dtype=dtype)
        self.layers = nn.ModuleList(
            [LolulornLayer(cfg, s, dtype,
                           a1_ranks.get(i, max(1, int(s["mixer"]["dim"]) // 2)))
             for i, s in enumerate(cfg.layers)])
        # cache stream of every attention layer: its own, or its source's
        self.stream_of, n = {}, 0
        for i, layer in enumerate(self.layers):
            if layer.kind == "attention" and layer.mixer.own_kv:
                self.stream_of[i] = n
                n += 1
        for i, layer in enumerate(self.layers):
            if layer.kind == "attention" and not layer.mixer.own_kv:
                self.stream_of[i] = self.stream_of[int(layer.mixer.kv_from)]
        self.final_norm = PostNorm(W, cfg.norm_eps)
        self.head = _w(cfg.vocab_size, W, dtype=dtype)

    # ------------------------------------------------------------ weights
    def init_random(self, seed=0):
        """Random weights of a useful scale for tests and benchmarks."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf == "weight" or leaf in ("q_norm", "k_norm", "norm"):
                p.data.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf in ("bias", "router_bias", "a2_bias", "dt_bias"):
                p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
            elif leaf == "a_log":
                p.data.copy_(torch.randn(p.shape, generator=g) - 1.0)
            elif leaf == "conv":
                p.data.copy_(0.4 * torch.randn(p.shape, generator=g))
            elif name == "embed":
                p.data.copy_(torch.randn(p.shape, generator=g))
            else:
                p.data.copy_(p.shape[-1] ** -0.5
                             * torch.randn(p.shape, generator=g))
        return self

    def load_named_tensors(self, t: dict):
        """Fill the parameters from tensors named as in the checkpoint
        (linear weights [out, in]; 'l<i>.mix.*', 'l<i>.mlp.*', ...)."""
        def put(p, v):
            if tuple(p.shape) != tuple(v.shape):
                raise ValueError(f"shape {tuple(v.shape)} != "
                                 f"{tuple(p.shape)}")
            p.data.copy_(v.to(p.dtype))

        put(self.embed, t["embed"])
        put(self.final_norm.weight, t["final.norm"])
        put(self.final_norm.bias, t["final.norm.b"])
        put(self.head, t["head"])
        for i, layer in enumerate(self.layers):
            pre, mp = f"l{i}.", f"l{i}.mix."
            a = layer.mixer
            put(layer.norm1.weight, t[pre + "norm1"])
            put(layer.norm1.bias, t[pre + "norm1.b"])
            if layer.kind == "attention":
                rows = [t[mp + "q"]]
                if a.own_kv:
                    rows += [t[mp + "k"], t[mp + "v"]]
                    put(a.k_norm, t[mp + "k.norm"])
                put(a.w_in, torch.cat(rows, 0))
                put(a.q_norm, t[mp + "q.norm"])
            elif layer.kind == "delta":
                put(a.w_in, torch.cat([t[mp + n] for n in "qkvgba"], 0))
                put(a.conv, torch.cat([t[mp + n + ".conv"] for n in "qkv"], 0))
                put(a.a_log, t[mp + "A_log"])
                put(a.dt_bias, t[mp + "dt_bias"])
                put(a.norm, t[mp + "norm"])
            else:
                put(a.w_in, torch.cat([t[mp + n] for n in
                                       ("q", "k", "v", "g", "a1")], 0))
                put(a.w_a2, t[mp + "a2"])
                put(a.a2_bias, t[mp + "a2.b"])
                put(a.norm, t[mp + "norm"])
            put(a.w_o, t[mp + "o"])
            m = layer.mlp
            if m is None:
                continue
            put(layer.norm2.weight, t[pre + "norm2"])
            put(layer.norm2.bias, t[pre + "norm2.b"])
            fp = pre + "mlp."
            if isinstance(m, GatedMLP):
                put(m.w_gu, torch.cat([t[fp + "gate"], t[fp + "up"]], 0))
                put(m.w_down, t[fp + "down"])
            else:
                put(m.router, t[fp + "router"])
                put(m.router_bias, t[fp + "correction"])
                put(m.w_gu, torch.stack(
                    [torch.cat([t[f"{fp}e{e}.gate"], t[f"{fp}e{e}.up"]], 0)
                     for e in range(m.experts)]))
                put(m.w_down, torch.stack([t[f"{fp}e{e}.down"]
                                           for e in range(m.experts)]))
        return self

    # -------------------------------------------------------------- cache
    def build_cache(self, max_slots, max_tokens, dtype=None, device=None,
                    block_size=64, **_):
        """One K/V row stream per attention layer that caches its own rows;
        per request slot the recurrent layers' matrix states (fp32) and
        convolution tails."""
        dtype = dtype or self.dtype
        device = device or self.embed.device
        dims = [self.layers[i].mixer.row_dim
                for i in sorted(self.stream_of, key=self.stream_of.get)
                if self.layers[i].mixer.own_kv]
        states = {}
        for i, layer in enumerate(self.layers):
            if layer.kind != "attention":
                for k, s in layer.mixer.state_shapes(dtype).items():
                    states[f"{k}{i}"] = s
        return PagedStateCache(dims, states, max_slots, max_tokens,
                               block_size=block_size, dtype=dtype,
                               device=device)

    # ------------------------------------------------------------ forward
    @torch.no_grad()
    def forward(self, input_ids, positions=None, kv_cache=None, rows=None,
                taps=None):
        """input_ids: flat [T] tokens of ``kv_cache.batch``. ``rows`` selects
        the flat positions whose logits are returned (default all).
        ``taps`` (a list) receives the stream after every layer."""
        cache = kv_cache
        assert cache is not None and cache.batch is not None, \
            "Lolulorn runs through a PagedStateCache step"
        ids = input_ids.reshape(-1)
        dt = self.dtype
        x = embed_rows(self.embed, ids, self.cfg.embed_scale)
        h = x if dt == torch.float32 else x.to(dt)
        for i, layer in enumerate(self.layers):
            states = {k: cache.states[f"{k}{i}"] for k in ("conv", "rec")
                      if f"{k}{i}" in cache.states}
            h = layer(x, h, cache, self.stream_of.get(i), states, dt)
            if taps is not None:
                taps.append(x.clone())
        n = self.final_norm
        return F.linear(layer_norm_rows(x, n.weight, n.bias, n.eps, dt, rows),
                        self.head)

    def num_parameters(self):
        return sum(p.numel() for p in self.parameters())


def build_from_config(cfg: dict, dtype, tensors=None):
    """Registry entry. Sizes that only the tensors give (the rank of the
    low-rank decay projection) are read from ``tensors`` when they are at
    hand."""
    ranks = {}
    for i, spec in enumerate(cfg["layers"]):
        key = f"l{i}.mix.a1"
        if spec["type"] == "gla":
            if tensors is not None and key in tensors:
                ranks[i] = int(tensors[key].shape[0])
            elif "rank" in spec["mixer"]:
                ranks[i] = int(spec["mixer"]["rank"])
    return LolulornForCausalLM(LolulornConfig.from_dict(cfg), dtype, ranks)


def lolulorn_tiny(dtype=torch.float32):
    """A small configuration for tests: every mixer kind, a shared K/V
    stream, a dense and a routed feed-forward."""
    att = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.4,
           "mask": {"size": 9, "keep_first": 2},
           "rot": {"base": 100.0, "dims": 4, "scaling": {"factor": 1.5}}}
    moe = {"kind": "moe", "expert": {"ff": 12},
           "router": {"experts": 6, "top": 2,
                      "groups": {"count": 3, "keep": 2}}}
    cfg = LolulornConfig(
        vocab_size=61, width=24, norm_eps=1e-5, embed_scale=3.0,
        layers=[{"type": "gla", "mixer": {"heads": 2, "dim": 6, "vdim": 8,
                                          "tau": 8.0},
                 "mlp": {"kind": "dense", "ff": 40}},
                {"type": "attention", "mixer": att, "mlp": moe},
                {"type": "attention", "mixer": {**att, "kv_from": 1},
                 "mlp": None},
                {"type": "delta", "mixer": {"heads": 4, "kv_heads": 2,
                                            "dim": 6, "vdim": 5, "conv": 3},
                 "mlp": moe}])
    return LolulornForCausalLM(cfg, dtype)
