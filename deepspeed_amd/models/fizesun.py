"""Fizesun: a decoder-only serving model assembled from the framework's
ragged-batch mechanisms.

* residual stream in fp32; every sublayer reads ``h + conv(h)`` where ``h``
  is a single-gain RMS norm of the stream and ``conv`` a short depthwise
  causal convolution with carried state (ops/causal_conv.py);
* mixer ``latent_attention``: compressed-KV attention over the paged cache
  with interleaved partial rotary and a per-head sigmoid output gate
  (ops/latent_attention.py);
* feed-forward: dense with the xIELU activation, or routed clamped-SwiGLU
  experts with an optional gated shared expert (moe/routed.py);
* a block of layers may be looped: it runs ``times`` passes over the same
  weights, each pass with cache streams of its own, entered through a
  projection of [stream ; embedding output] plus a per-pass offset.

The model runs only through a ``PagedStateCache``: ``forward`` takes the flat
token list of a ragged batch. All sizes and constants come from the config.
"""

from dataclasses import dataclass, field
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..inference.state_cache import PagedStateCache
from ..moe.routed import RoutedExperts
from ..ops.activations import xielu
from ..ops.causal_conv import norm_conv_ragged, residual_add_stats
from ..ops.latent_attention import (gate_merge_heads, latent_attention,
                                    latent_prep)
from ..ops.norms import ScalarRMSNorm
from ..ops.rope import rope_tables


@dataclass
class FizesunConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6
    conv_taps: int = 4
    loop: Optional[dict] = None          # {"start", "stop", "times"}
    max_seq_len: int = 1 << 16           # rotary table growth bound
    extra: dict = field(default_factory=dict)

    @classmethod
    def from_dict(cls, d: dict) -> "FizesunConfig":
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]),
                   layers=list(d["layers"]),
                   norm_eps=float(d["norm"]["eps"]),
                   conv_taps=int(d["canon"]["taps"]),
                   loop=d.get("loop") or None)

    def to_dict(self) -> dict:
        d = {"architecture": "Fizesun", "vocab": self.vocab_size,
             "width": self.width, "layers": self.layers,
             "norm": {"eps": self.norm_eps},
             "canon": {"taps": self.conv_taps}}
        if self.loop:
            d["loop"] = self.loop
        return d

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def layer_runs(self):
        """[(layer, pass or None, enters_pass)] in execution order; the index
        in this list is the layer run's cache stream."""
        n = len(self.layers)
        if not self.loop:
            return [(i, None, False) for i in range(n)]
        a, b, times = (int(self.loop[k]) for k in ("start", "stop", "times"))
        runs = [(i, None, False) for i in range(a)]
        for t in range(times):
            runs += [(i, t, i == a) for i in range(a, b)]
        return runs + [(i, None, False) for i in range(b, n)]


def _w(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


class LatentAttention(nn.Module):
    """Input projection fused as [q | latent | k_rot | gate] rows; the key and
    value up-projections are kept per head for folding into q and the
    output."""

    def __init__(self, width, m: dict, eps, dtype):
        super().__init__()
        self.heads, self.dim, self.rot = m["heads"], m["dim"], m["rot_dim"]
        self.vdim, self.rank = m["vdim"], m["kv_rank"]
        self.rot_dims = int(m["rot"]["dims"])
        self.rot_base = float(m["rot"]["base"])
        self.scale = float(m["scale"])
        self.eps = eps
        H = self.heads
        rows = H * (self.dim + self.rot) + self.rank + self.rot + H
        self.w_in = _w(rows, width, dtype=dtype)
        self.latent_norm = _w(self.rank, dtype=torch.float32)
        self.w_uk = _w(H, self.dim, self.rank, dtype=dtype)    # q_nope -> rank
        self.w_uv = _w(H, self.rank, self.vdim, dtype=dtype)   # rank -> v
        self.w_o = _w(width, H * self.vdim, dtype=dtype)

    @property
    def row_dim(self):
        return self.rank + self.rot

    def forward(self, h, cache: PagedStateCache, stream: int, max_pos: int):
        b = cache.batch
        cos, sin = rope_tables(self.rot_dims, max_pos, self.rot_base,
                               device=h.device)
        pool = cache.pools[stream]
        q_nope, q_rot, gate = latent_prep(
            F.linear(h, self.w_in), b, pool, self.latent_norm, self.eps,
            self.heads, self.dim, self.rot, self.rank, self.rot_dims, cos,
            sin)
        q_lat = torch.bmm(q_nope, self.w_uk)                  # [H, T, rank]
        o_lat = latent_attention(q_lat, q_rot, pool, b, self.rank, self.scale)
        o = torch.bmm(o_lat, self.w_uv)                       # [H, T, vdim]
        return F.linear(gate_merge_heads(o, gate), self.w_o)


class XieluMLP(nn.Module):
    def __init__(self, width, ff, dtype):
        super().__init__()
        self.w_up = _w(ff, width, dtype=dtype)
        self.w_down = _w(width, ff, dtype=dtype)
        self.act = _w(2, dtype=torch.float32)

    def forward(self, h):
        return F.linear(xielu(F.linear(h, self.w_up), self.act), self.w_down)


class FizesunLayer(nn.Module):
    def __init__(self, cfg: FizesunConfig, spec: dict, dtype):
        super().__init__()
        W, taps = cfg.width, cfg.conv_taps
        if spec["type"] != "latent_attention":
            raise ValueError(f"unknown mixer type {spec['type']!r}")
        self.norm1 = ScalarRMSNorm(cfg.norm_eps)
        self.conv1 = _w(W, taps, dtype=dtype)
        self.mixer = LatentAttention(W, spec["mixer"], cfg.norm_eps, dtype)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp:
            self.norm2 = ScalarRMSNorm(cfg.norm_eps)
            self.conv2 = _w(W, taps, dtype=dtype)
            if mlp["kind"] == "dense":
                self.mlp = XieluMLP(W, mlp["ff"], dtype)
            elif mlp["kind"] == "moe":
                sh = mlp.get("shared") or {}
                self.mlp = RoutedExperts(
                    W, mlp["expert"]["ff"], mlp["router"]["experts"],
                    mlp["router"]["top"], mlp["expert"]["limit"],
                    shared_ff=sh.get("ff", 0),
                    shared_limit=sh.get("limit", 0.0), dtype=dtype)
            else:
                raise ValueError(f"unknown mlp kind {mlp['kind']!r}")

    def forward(self, x, cache, stream, dtype, max_pos, sumsq=None):
        """x: fp32 stream, updated in place. ``sumsq``: row sums of squares of
        x when its producer computed them. Returns the sums of the new x (or
        None) for the next layer's first norm."""
        b = cache.batch
        h = norm_conv_ragged(x, self.norm1.gain, self.norm1.eps, self.conv1,
                             cache.states["conv"][:, 2 * stream], b, dtype,
                             sumsq)
        sumsq = residual_add_stats(x, self.mixer(h, cache, stream, max_pos))
        if self.mlp is not None:
            h = norm_conv_ragged(x, self.norm2.gain, self.norm2.eps,
                                 self.conv2,
                                 cache.states["conv"][:, 2 * stream + 1], b,
                                 dtype, sumsq)
            sumsq = residual_add_stats(x, self.mlp(h))
        return sumsq


class FizesunForCausalLM(nn.Module):
    architecture = "Fizesun"

    def __init__(self, cfg: FizesunConfig, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        W = cfg.width
        self.embed = _w(cfg.vocab_size, W, dtype=dtype)
        self.embed_norm = ScalarRMSNorm(cfg.norm_eps)
        self.layers = nn.ModuleList(
            [FizesunLayer(cfg, s, dtype) for s in cfg.layers])
        self.runs = cfg.layer_runs()
        if cfg.loop:
            self.loop_in = _w(W, 2 * W, dtype=dtype)
            self.loop_step = _w(int(cfg.loop["times"]), W,
                                dtype=torch.float32)
        self.final_norm = ScalarRMSNorm(cfg.norm_eps)
        self.head = _w(cfg.vocab_size, W, dtype=dtype)

    # ------------------------------------------------------------ weights
    def init_random(self, seed=0, std=None):
        """Random weights of a useful scale for tests and benchmarks."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            if name.endswith(".gain"):
                p.data.fill_(1.0)
            elif name.endswith("latent_norm"):
                p.data.copy_(1 + 0.1 * torch.randn(p.shape, generator=g))
            elif name.endswith(".act") or name.endswith("router_bias") \
                    or name == "loop_step":
                p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
            elif "conv" in name:
                p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
            elif name == "embed":
                p.data.copy_(torch.randn(p.shape, generator=g))
            else:
                s = std or p.shape[-1] ** -0.5
                p.data.copy_(s * torch.randn(p.shape, generator=g))
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
        put(self.embed_norm.gain, t["embed.norm"].reshape(1))
        put(self.final_norm.gain, t["final.norm"].reshape(1))
        put(self.head, t["head"])
        if self.cfg.loop:
            put(self.loop_in, t["loop.in"])
            put(self.loop_step, t["loop.step"])
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            a = layer.mixer
            put(layer.norm1.gain, t[pre + "norm1"].reshape(1))
            put(layer.conv1, t[pre + "canon1"])
            put(a.w_in, torch.cat([t[pre + "mix.q"], t[pre + "mix.dkv"],
                                   t[pre + "mix.g"]], 0))
            put(a.latent_norm, t[pre + "mix.dkv.norm"])
            put(a.w_uk, t[pre + "mix.uk"].reshape(a.heads, a.dim, a.rank))
            put(a.w_uv, t[pre + "mix.uv"].reshape(a.heads, a.vdim, a.rank)
                .transpose(1, 2))
            put(a.w_o, t[pre + "mix.o"])
            m = layer.mlp
            if m is None:
                continue
            put(layer.norm2.gain, t[pre + "norm2"].reshape(1))
            put(layer.conv2, t[pre + "canon2"])
            mp = pre + "mlp."
            if isinstance(m, XieluMLP):
                put(m.w_up, t[mp + "up"])
                put(m.w_down, t[mp + "down"])
                put(m.act, t[mp + "act"])
            else:
                put(m.router, t[mp + "router"])
                put(m.router_bias, t[mp + "router.b"])
                put(m.w_gu, torch.stack(
                    [torch.cat([t[f"{mp}e{e}.gate"], t[f"{mp}e{e}.up"]], 0)
                     for e in range(m.experts)]))
                put(m.w_down, torch.stack([t[f"{mp}e{e}.down"]
                                           for e in range(m.experts)]))
                if m.shared is not None:
                    put(m.shared.w_gu, torch.cat([t[mp + "shared.gate"],
                                                  t[mp + "shared.up"]], 0))
                    put(m.shared.w_down, t[mp + "shared.down"])
                    put(m.shared_gate, t[mp + "shared.sg"])
        return self

    # -------------------------------------------------------------- cache
    def build_cache(self, max_slots, max_tokens, dtype=None, device=None,
                    block_size=64, **_):
        """The cache manager this design needs: one row stream per layer run
        and the convolution tails of both sublayers of every run."""
        dtype = dtype or self.dtype
        device = device or self.embed.device
        dims = [self.layers[i].mixer.row_dim for i, _, _ in self.runs]
        tail = max(self.cfg.conv_taps - 1, 0)
        states = {"conv": (2 * len(self.runs), tail, self.cfg.width)}
        return PagedStateCache(dims, states, max_slots, max_tokens,
                               block_size=block_size, dtype=dtype,
                               device=device)

    # ------------------------------------------------------------ forward
    @torch.no_grad()
    def forward(self, input_ids, positions=None, kv_cache=None, rows=None,
                taps=None):
        """input_ids: flat [T] tokens of ``kv_cache.batch``. ``rows`` selects
        the flat positions whose logits are returned (default all).
        ``taps`` (a list) receives the stream after every layer run."""
        cache = kv_cache
        assert cache is not None and cache.batch is not None, \
            "Fizesun runs through a PagedStateCache step"
        ids = input_ids.reshape(-1)
        dt = self.dtype
        max_pos = cache.max_seq
        x0 = self.embed_norm(self.embed, out_dtype=torch.float32, index=ids)
        x = x0.clone()
        sumsq = None
        for stream, (i, t, enters) in enumerate(self.runs):
            if enters:
                x = F.linear(torch.cat([x, x0], -1).to(dt), self.loop_in) \
                    .float().add_(self.loop_step[t])
                sumsq = None
            sumsq = self.layers[i](x, cache, stream, dt, max_pos, sumsq)
            if taps is not None:
                taps.append(x.clone())
        return F.linear(self.final_norm(x, out_dtype=dt, index=rows),
                        self.head)

    def num_parameters(self):
        return sum(p.numel() for p in self.parameters())


def fizesun_tiny(dtype=torch.float32):
    """A small configuration for tests: two attention shapes, a dense and a
    routed feed-forward, a looped block."""
    mix = {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 12,
           "rot": {"base": 100.0, "dims": 4}, "scale": 12 ** -0.5}
    cfg = FizesunConfig(
        vocab_size=67, width=24, norm_eps=1e-5, conv_taps=3,
        loop={"start": 0, "stop": 1, "times": 2},
        layers=[{"type": "latent_attention", "mixer": mix,
                 "mlp": {"kind": "dense", "ff": 40}},
                {"type": "latent_attention", "mixer": mix,
                 "mlp": {"kind": "moe", "expert": {"ff": 16, "limit": 1.5},
                         "router": {"experts": 5, "top": 2},
                         "shared": {"ff": 8, "limit": 2.5}}}])
    return FizesunForCausalLM(cfg, dtype)
