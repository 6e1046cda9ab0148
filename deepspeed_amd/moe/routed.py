"""Serving-side mixture of experts: no capacity, no token dropping.

``topk_softmax`` picks each token's ``top`` largest router logits and weights
them by a softmax over the CHOSEN logits only (fp32). ``RoutedExperts`` runs
clamped-SwiGLU experts: tokens are grouped by expert, each expert is one pair
of vendor GEMMs on its contiguous group, and a combine kernel sums a token's
weighted expert outputs (plus an optional shared expert scaled by a per-token
sigmoid gate) in fp32. Training-time MoE with capacity and all-to-all lives
in sharded_moe.py.
"""

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops.activations import clamped_swiglu


def _sk():
    from ..ops import serving_kernels
    return serving_kernels


def topk_softmax(logits, top):
    """logits [T, E] fp32 -> (idx [T, top] int64, weight [T, top] fp32)."""
    if logits.is_cuda and _sk().enabled():
        return _sk().topk_softmax(logits.float(), top)
    val, idx = torch.topk(logits.float(), top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def moe_combine(y, inv, weight, shared=None, shared_gate=None):
    """y [N, C] expert outputs; inv [T, top] the row of y that holds each
    (token, choice); weight [T, top] fp32. Returns
    sum_k weight[t, k] * y[inv[t, k]] (+ sigmoid(shared_gate[t]) *
    shared[t]) as [T, C] in y's dtype."""
    if y.is_cuda and _sk().enabled():
        sk = _sk()
        return sk.moe_combine(y, inv, weight, shared, shared_gate)
    out = (y.float()[inv] * weight[..., None]).sum(1)
    if shared is not None:
        out = out + torch.sigmoid(shared_gate.float()) * shared.float()
    return out.to(y.dtype)


class ClampedGLUExpert(nn.Module):
    """down(clamped_swiglu([gate; up] h)) without biases."""

    def __init__(self, width, ff, limit, dtype=torch.float32):
        super().__init__()
        self.limit = float(limit)
        self.w_gu = nn.Parameter(torch.empty(2 * ff, width, dtype=dtype),
                                 requires_grad=False)
        self.w_down = nn.Parameter(torch.empty(width, ff, dtype=dtype),
                                   requires_grad=False)

    def forward(self, h):
        return F.linear(clamped_swiglu(F.linear(h, self.w_gu), self.limit),
                        self.w_down)


class RoutedExperts(nn.Module):
    def __init__(self, width, ff, experts, top, limit, shared_ff=0,
                 shared_limit=0.0, dtype=torch.float32):
        super().__init__()
        self.experts, self.top, self.limit = experts, top, float(limit)
        self.router = nn.Parameter(torch.empty(experts, width,
                                               dtype=torch.float32),
                                   requires_grad=False)
        self.router_bias = nn.Parameter(torch.zeros(experts,
                                                    dtype=torch.float32),
                                        requires_grad=False)
        self.w_gu = nn.Parameter(torch.empty(experts, 2 * ff, width,
                                             dtype=dtype), requires_grad=False)
        self.w_down = nn.Parameter(torch.empty(experts, width, ff,
                                               dtype=dtype),
                                   requires_grad=False)
        self.shared = None
        if shared_ff:
            self.shared = ClampedGLUExpert(width, shared_ff, shared_limit,
                                           dtype)
            self.shared_gate = nn.Parameter(torch.empty(1, width, dtype=dtype),
                                            requires_grad=False)

    def forward(self, h):
        T = h.shape[0]
        logits = F.linear(h.float(), self.router.float(),
                          self.router_bias.float())
        idx, weight = topk_softmax(logits, self.top)
        picks = T * self.top
        if picks <= self.DENSE_MAX_PICKS and 2 * picks >= self.experts:
            # decode-sized steps: run every expert on every token as three
            # batched GEMMs (the picks of a few tokens touch most experts'
            # weights anyway) and pick the chosen outputs; no host round trip
            mid = clamped_swiglu(torch.bmm(h.expand(self.experts, T, -1),
                                           self.w_gu.transpose(1, 2)),
                                 self.limit)
            y = torch.bmm(mid, self.w_down.transpose(1, 2)) \
                .reshape(self.experts * T, -1)
            inv = idx * T + torch.arange(T, device=h.device)[:, None]
        else:
            y, inv = self._grouped(h, idx)
        sh = sg = None
        if self.shared is not None:
            sh = self.shared(h)
            sg = F.linear(h, self.shared_gate)
        return moe_combine(y, inv, weight, sh, sg)

    DENSE_MAX_PICKS = 64

    def _grouped(self, h, idx):
        """Tokens sorted by expert; one pair of GEMMs per expert that has
        tokens. Returns the outputs in sorted order and each pick's place."""
        T = h.shape[0]
        flat = idx.reshape(-1)
        order = torch.argsort(flat, stable=True)
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        counts = torch.bincount(flat, minlength=self.experts).tolist()
        xs = h[order // self.top]
        y = torch.empty(T * self.top, h.shape[1], dtype=h.dtype,
                        device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                mid = clamped_swiglu(F.linear(xs[at:at + n], self.w_gu[e]),
                                     self.limit)
                y[at:at + n] = F.linear(mid, self.w_down[e])
                at += n
        return y, inv.view(T, self.top)
