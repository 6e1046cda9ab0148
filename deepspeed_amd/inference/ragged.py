"""Continuous batching over a slotted KV pool — FastGen-lite (reference:
deepspeed/inference/v2 engine_v2.py put/query :107-184, ragged KV cache,
Dynamic SplitFuse scheduling).

Sequences of different lengths decode together: each live request owns a
SLOT of a pre-allocated per-layer KV pool; one model step advances every
active sequence by one token (new requests are prefilled into their slot
as they arrive). The per-slot positions differ, so attention uses an
explicit validity mask instead of `is_causal` — the mask is produced by
``RaggedKVCache`` and consumed by the model via ``kv_cache.last_mask``.

Design delta vs the reference: no paged blocks — 288 GB of HBM3E holds a
contiguous max_seq slot per request for any single-node serving
configuration, which keeps KV reads fully coalesced and the scheduler
trivial (a free-slot list).
"""

from collections import deque
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


class RaggedKVCache:
    """Slot-pooled KV: [slots, Hkv, max_seq, D] per layer + per-slot
    lengths. ``begin_step(slots, q_len)`` selects the active batch; the
    following per-layer ``update`` calls write at each slot's own cursor
    and return padded K/V plus the validity mask."""

    def __init__(self, num_layers: int, num_slots: int, kv_heads: int,
                 max_seq: int, head_dim: int, dtype=torch.float32,
                 device="cpu"):
        shape = (num_slots, kv_heads, max_seq, head_dim)
        self.k = [torch.zeros(shape, dtype=dtype, device=device)
                  for _ in range(num_layers)]
        self.v = [torch.zeros(shape, dtype=dtype, device=device)
                  for _ in range(num_layers)]
        self.lens = torch.zeros(num_slots, dtype=torch.long, device=device)
        self.max_seq = max_seq
        self.device = device
        self._slots: Optional[torch.Tensor] = None
        self._q_len = 0
        self.last_mask: Optional[torch.Tensor] = None

    def free(self, slot: int):
        self.lens[slot] = 0

    def begin_step(self, slots: List[int], q_len: int, offsets=None):
        """All sequences in this step share q_len (1 for decode; the prompt
        length for a single-sequence prefill). SplitFuse token packing:
        pass q_len=1 with one entry per TOKEN — `slots` may repeat and
        `offsets[i]` places token i at ``lens[slot]+offsets[i]``, so a
        prefill chunk and the decode batch ride one forward."""
        self._slots = torch.as_tensor(slots, dtype=torch.long,
                                      device=self.device)
        self._q_len = q_len
        self._packed = offsets is not None
        starts = self.lens[self._slots]             # [n]
        if self._packed:
            assert q_len == 1, "packed mode is per-token (q_len 1)"
            starts = starts + torch.as_tensor(offsets, dtype=torch.long,
                                              device=self.device)
        n = len(slots)
        L = int((starts + q_len).max())
        # mask[i, 1, qi, j]: query at absolute pos starts_i+qi may see j
        pos = torch.arange(L, device=self.device)
        qpos = starts[:, None, None] + torch.arange(q_len,
                                                    device=self.device)[None, :,
                                                                        None]
        self.last_mask = (pos[None, None, :] <= qpos).unsqueeze(1)  # [n,1,q,L]
        self._L = L
        self._starts = starts

    def update(self, layer_idx: int, k: torch.Tensor, v: torch.Tensor):
        """k, v: [n, Hkv, q_len, D] -> padded ([n, Hkv, L, D], same)."""
        n, Hkv, q_len, D = k.shape
        assert q_len == self._q_len
        sl = self._slots
        for j in range(q_len):  # q_len==1 in steady decode
            self.k[layer_idx][sl, :, self._starts + j] = k[:, :, j]
            self.v[layer_idx][sl, :, self._starts + j] = v[:, :, j]
        return (self.k[layer_idx][sl, :, :self._L],
                self.v[layer_idx][sl, :, :self._L])

    def end_step(self):
        if self._packed:   # repeated slots: one token each
            self.lens.index_add_(0, self._slots,
                                 torch.ones_like(self._slots))
        else:
            self.lens[self._slots] += self._q_len
        self._slots = None
        self.last_mask = None


@dataclass
class Request:
    uid: int
    prompt: torch.Tensor                      # [S] token ids
    max_new_tokens: int = 64
    eos_token_id: Optional[int] = None
    # per-request sampling params (reference inference/v2 SamplingParams)
    do_sample: bool = False
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    slot: int = -1
    prefilled: int = 0                        # prompt tokens already in KV
    generated: List[int] = field(default_factory=list)
    done: bool = False

    def select(self, logits: torch.Tensor) -> int:
        from .engine import _select_token
        return int(_select_token(logits.view(1, -1), self.do_sample,
                                 self.temperature, self.top_k, self.top_p))

    @property
    def in_prefill(self) -> bool:
        return self.prefilled < self.prompt.numel()

    @property
    def tokens(self) -> List[int]:
        return self.prompt.tolist() + self.generated


class ContinuousBatcher:
    """Iteration-level scheduler: every call to step() (1) prefills queued
    requests into free slots, (2) advances all active sequences one token
    in a single batched forward (reference engine_v2 put/schedule loop)."""

    def __init__(self, model, max_slots: int = 8, max_seq: int = None,
                 dtype=torch.float32, device=None,
                 prefill_chunk: int = 0, cache_cls=None,
                 token_budget: int = 0, max_tokens: int = 0):
        """``prefill_chunk`` > 0 bounds prompt tokens prefetched per step
        (Dynamic SplitFuse: long prompts stream in across iterations so the
        decode batch's latency stays flat; reference inference/v2
        scheduling). 0 = whole prompt in one step.

        ``token_budget`` > 0 enables TRUE SplitFuse token packing: every
        iteration issues ONE forward whose batch rows are individual
        tokens — the whole decode batch plus up to the remaining budget of
        prefill-chunk tokens — so prefill never stalls decode and each
        step's work is a constant ~token_budget tokens (reference Dynamic
        SplitFuse scheduling, inference/v2).

        ``max_tokens`` sizes a model-provided paged cache: the most tokens
        live at once, each request rounded up to whole blocks (default
        ``max_slots * max_seq``)."""
        self.model = model
        cfg = model.cfg
        self.device = device or next(model.parameters()).device
        max_seq = max_seq or cfg.max_seq_len
        # A model whose layers cache something other than per-head K/V
        # brings its own manager (``build_cache``); such caches describe a
        # step as a flat ragged batch instead of padded rows + mask.
        self.ragged = hasattr(model, "build_cache")
        if self.ragged:
            self.cache = model.build_cache(
                max_slots, max_tokens or max_slots * max_seq, dtype=dtype,
                device=self.device)
            if token_budget <= 0:
                token_budget = 2048
        else:
            kv_heads = getattr(cfg, "num_kv_heads", None) or cfg.num_heads
            cache_cls = cache_cls or RaggedKVCache
            self.cache = cache_cls(cfg.num_layers, max_slots, kv_heads,
                                   max_seq, cfg.head_dim, dtype=dtype,
                                   device=self.device)
        self.free_slots = deque(range(max_slots))
        self.pending: deque = deque()
        self.active: Dict[int, Request] = {}
        self.prefill_chunk = prefill_chunk
        self.token_budget = token_budget

    def put(self, req: Request):
        self.pending.append(req)

    def has_work(self) -> bool:
        return bool(self.pending or self.active)

    @torch.no_grad()
    def _forward(self, ids, slots, q_len, positions):
        self.cache.begin_step(slots, q_len)
        logits = self.model(ids, positions=positions, kv_cache=self.cache)
        self.cache.end_step()
        return logits

    def _prefill_some(self, req: Request):
        """Advance one request's prefill by up to prefill_chunk tokens; on
        completion, sample its first token."""
        S = req.prompt.numel()
        chunk = S - req.prefilled if self.prefill_chunk <= 0 \
            else min(self.prefill_chunk, S - req.prefilled)
        lo, hi = req.prefilled, req.prefilled + chunk
        pos = torch.arange(lo, hi, dtype=torch.int32,
                           device=self.device).unsqueeze(0)
        logits = self._forward(
            req.prompt[lo:hi].view(1, -1).to(self.device), [req.slot],
            chunk, pos)
        req.prefilled = hi
        if not req.in_prefill:
            req.generated.append(req.select(logits[0, -1]))

    def _admit(self):
        while self.pending and self.free_slots:
            if self.ragged and not self._fits(self.pending[0]):
                break        # wait for blocks; keeps arrival order
            req = self.pending.popleft()
            self._take_slot(req)

    def _take_slot(self, req: Request):
        req.slot = self.free_slots.popleft()
        if self.ragged:
            self.cache.reset_slot(req.slot)
        else:
            self.cache.free(req.slot)
            self.cache.lens[req.slot] = 0
        self.active[req.uid] = req

    def _blocks_for(self, req: Request) -> int:
        bs = self.cache.block_size
        return (req.prompt.numel() + req.max_new_tokens + bs - 1) // bs

    def _fits(self, req: Request) -> bool:
        """Admission control for a paged pool: a request enters only if the
        blocks it can grow to are not promised to the live ones."""
        promised = sum(self._blocks_for(r) for r in self.active.values())
        return promised + self._blocks_for(req) <= self.cache.num_blocks

    # ------------------------------------------------ externally driven steps
    def open(self, uid, max_new_tokens: int = 0) -> Request:
        """Admit a request whose tokens the caller feeds step by step
        (replaying a recorded schedule, speculative drivers, tests)."""
        assert self.ragged, "open/feed/close need a ragged cache"
        if not self.free_slots:
            raise RuntimeError("no free request slot")
        req = Request(uid=uid, prompt=torch.empty(0, dtype=torch.long),
                      max_new_tokens=max_new_tokens)
        self._take_slot(req)
        return req

    @torch.no_grad()
    def feed(self, entries, rows=None):
        """ONE model step over a ragged batch: ``entries`` is a list of
        (request, tokens) — a prompt portion for some, one decoded token for
        others. Returns logits for the flat token positions ``rows`` (default:
        every token). This is the step the scheduler itself runs."""
        slots = [r.slot for r, _ in entries]
        counts = [len(t) for _, t in entries]
        ids = torch.tensor([int(x) for _, t in entries for x in t],
                           dtype=torch.long).to(self.device)
        self.cache.begin_ragged(slots, counts)
        try:
            if rows is not None:
                rows = torch.as_tensor(rows, dtype=torch.long).to(self.device)
            logits = self.model(ids, kv_cache=self.cache, rows=rows)
        finally:
            self.cache.end_step()
        return logits

    def close(self, req: Request):
        """Give a request's slot and blocks back."""
        req.done = True
        self.cache.free(req.slot)
        self.free_slots.append(req.slot)
        self.active.pop(req.uid, None)

    @torch.no_grad()
    def _step_ragged(self) -> List[Request]:
        """Token-budgeted iteration on a ragged cache: every decoding request
        contributes its last token, prompts fill the rest of the budget in
        portions; one forward for all of it."""
        self._admit()
        finished = self._retire()
        entries, budget = [], self.token_budget
        for r in self.active.values():
            if not r.in_prefill:
                entries.append((r, [r.generated[-1]], 0))
                budget -= 1
        for r in self.active.values():
            if r.in_prefill and budget > 0:
                chunk = min(budget, r.prompt.numel() - r.prefilled)
                if self.prefill_chunk > 0:
                    chunk = min(chunk, self.prefill_chunk)
                entries.append(
                    (r, r.prompt[r.prefilled:r.prefilled + chunk].tolist(),
                     chunk))
                budget -= chunk
        if not entries:
            return finished
        last, at, sampled = [], 0, []
        for r, toks, chunk in entries:
            at += len(toks)
            if chunk == 0 or r.prefilled + chunk == r.prompt.numel():
                last.append(at - 1)
                sampled.append(r)
        logits = self.feed([(r, t) for r, t, _ in entries], rows=last) \
            if last else self.feed([(r, t) for r, t, _ in entries], rows=[0])
        for r, _, chunk in entries:
            r.prefilled += chunk
        for i, r in enumerate(sampled):
            r.generated.append(r.select(logits[i]))
        return finished

    def _retire(self) -> List[Request]:
        finished = []
        for uid in list(self.active):
            req = self.active[uid]
            if req.in_prefill:
                continue
            if (req.eos_token_id is not None and req.generated and
                    req.generated[-1] == req.eos_token_id) or \
                    len(req.generated) >= req.max_new_tokens or \
                    int(self.cache.lens[req.slot]) + 1 >= self.cache.max_seq:
                req.done = True
                finished.append(req)
                self.cache.free(req.slot)   # return KV blocks to the pool
                self.free_slots.append(req.slot)
                del self.active[uid]
        return finished

    @torch.no_grad()
    def _step_packed(self) -> List[Request]:
        """True SplitFuse iteration: one forward, batch rows = tokens."""
        self._admit()
        finished = self._retire()
        slots, offsets, ids, owners = [], [], [], []
        budget = self.token_budget
        for r in self.active.values():      # decodes first — latency
            if not r.in_prefill:
                slots.append(r.slot)
                offsets.append(0)
                ids.append(r.generated[-1])
                owners.append((r, 0))
                budget -= 1
        for r in self.active.values():      # fill with prefill chunks
            if budget <= 0:
                break
            if r.in_prefill:
                chunk = min(budget, r.prompt.numel() - r.prefilled)
                if self.prefill_chunk > 0:
                    chunk = min(chunk, self.prefill_chunk)
                for j in range(chunk):
                    slots.append(r.slot)
                    offsets.append(j)
                    ids.append(int(r.prompt[r.prefilled + j]))
                owners.append((r, chunk))
                budget -= chunk
        if not slots:
            return finished
        T = len(slots)
        ids_t = torch.tensor(ids, device=self.device).view(T, 1)
        lens = self.cache.lens
        pos = (lens[torch.as_tensor(slots, device=lens.device)] +
               torch.as_tensor(offsets, device=lens.device)).to(
                   device=self.device, dtype=torch.int32).view(T, 1)
        self.cache.begin_step(slots, 1, offsets=offsets)
        logits = self.model(ids_t, positions=pos, kv_cache=self.cache)
        self.cache.end_step()
        row = 0
        for r, chunk in owners:
            if chunk == 0:                       # decode row
                r.generated.append(r.select(logits[row, -1]))
                row += 1
            else:                                # prefill rows
                row += chunk
                r.prefilled += chunk
                if not r.in_prefill:             # prompt complete: sample
                    r.generated.append(r.select(logits[row - 1, -1]))
        return finished

    @torch.no_grad()
    def step(self) -> List[Request]:
        """One scheduling iteration; returns requests finished this step."""
        if self.ragged:
            return self._step_ragged()
        if self.token_budget > 0:
            return self._step_packed()
        # 1) admit queued requests into free slots
        self._admit()
        # 1b) advance prefills (bounded per step when prefill_chunk is set)
        for req in self.active.values():
            if req.in_prefill:
                self._prefill_some(req)

        # 2) retire sequences that hit eos/max BEFORE the decode batch
        finished = self._retire()

        # 3) one batched decode step for every fully-prefilled sequence
        decode = [r for r in self.active.values() if not r.in_prefill]
        if decode:
            reqs = decode
            slots = [r.slot for r in reqs]
            last = torch.tensor([[r.generated[-1]] for r in reqs],
                                device=self.device)
            lens = self.cache.lens
            idx = torch.as_tensor(slots, device=lens.device)
            pos = lens[idx].to(device=self.device,
                               dtype=torch.int32).unsqueeze(1)
            logits = self._forward(last, slots, 1, pos)
            for i, r in enumerate(reqs):
                r.generated.append(r.select(logits[i, -1]))
        return finished

    @torch.no_grad()
    def run_to_completion(self, max_steps: int = 10_000) -> List[Request]:
        out = []
        for _ in range(max_steps):
            if not self.has_work():
                break
            out.extend(self.step())
        return out


class PagedKVCache:
    """Blocked KV cache (reference: inference/v2/ragged blocked KV +
    csrc block allocator): storage is a shared pool of fixed-size blocks
    [num_blocks, Hkv, block_size, D]; each slot owns a growable block list,
    so HBM is committed per ~block instead of per max_seq slot. Same
    begin_step/update/end_step protocol as RaggedKVCache, so it drops into
    ContinuousBatcher unchanged; reads materialize the active slots'
    blocks into a padded [n, Hkv, L, D] view per step."""

    def __init__(self, num_layers: int, num_slots: int, kv_heads: int,
                 max_seq: int, head_dim: int, dtype=torch.float32,
                 device="cpu", block_size: int = 64, num_blocks: int = None):
        self.block_size = block_size
        blocks_per_slot = (max_seq + block_size - 1) // block_size
        self.num_blocks = num_blocks or num_slots * blocks_per_slot
        shape = (self.num_blocks, kv_heads, block_size, head_dim)
        self.k = [torch.zeros(shape, dtype=dtype, device=device)
                  for _ in range(num_layers)]
        self.v = [torch.zeros(shape, dtype=dtype, device=device)
                  for _ in range(num_layers)]
        self.free_blocks = list(range(self.num_blocks - 1, -1, -1))
        self.block_table: Dict[int, List[int]] = {s: [] for s in
                                                  range(num_slots)}
        self.lens = torch.zeros(num_slots, dtype=torch.long)
        self.max_seq = max_seq
        self.device = device
        self.last_mask: Optional[torch.Tensor] = None

    def free(self, slot: int):
        self.free_blocks.extend(reversed(self.block_table[slot]))
        self.block_table[slot] = []
        self.lens[slot] = 0

    def _ensure_blocks(self, slot: int, upto: int):
        need = (upto + self.block_size - 1) // self.block_size
        while len(self.block_table[slot]) < need:
            assert self.free_blocks, "paged KV pool exhausted"
            self.block_table[slot].append(self.free_blocks.pop())

    def begin_step(self, slots: List[int], q_len: int, offsets=None):
        self._slots = list(slots)
        self._q_len = q_len
        self._packed = offsets is not None
        starts = self.lens[torch.as_tensor(self._slots,
                                           device=self.lens.device)]
        if self._packed:
            assert q_len == 1, "packed mode is per-token (q_len 1)"
            starts = starts + torch.as_tensor(offsets,
                                              device=self.lens.device)
        L = int((starts + q_len).max())
        for s, st in zip(self._slots, starts.tolist()):
            self._ensure_blocks(s, st + q_len)
        pos = torch.arange(L, device=self.device)
        qpos = (starts.to(self.device)[:, None, None] +
                torch.arange(q_len, device=self.device)[None, :, None])
        self.last_mask = (pos[None, None, :] <= qpos).unsqueeze(1)
        self._L = L
        self._starts = starts

    def update(self, layer_idx: int, k: torch.Tensor, v: torch.Tensor):
        n, Hkv, q_len, D = k.shape
        bs = self.block_size
        for i, s in enumerate(self._slots):
            st = int(self._starts[i])
            for j in range(q_len):
                p = st + j
                blk = self.block_table[s][p // bs]
                self.k[layer_idx][blk, :, p % bs] = k[i, :, j]
                self.v[layer_idx][blk, :, p % bs] = v[i, :, j]
        # materialize padded views: gather each slot's blocks
        nblk = (self._L + bs - 1) // bs
        idx = torch.tensor([ (self.block_table[s] + [0] * nblk)[:nblk]
                             for s in self._slots ], dtype=torch.long,
                           device=self.device)              # [n, nblk]
        kb = self.k[layer_idx][idx]                          # [n,nblk,Hkv,bs,D]
        vb = self.v[layer_idx][idx]
        kb = kb.permute(0, 2, 1, 3, 4).reshape(n, Hkv, nblk * bs, D)
        vb = vb.permute(0, 2, 1, 3, 4).reshape(n, Hkv, nblk * bs, D)
        return kb[:, :, :self._L], vb[:, :, :self._L]

    def decode_attention(self, layer_idx: int, q, k, v, scale=None):
        """Single-token decode THROUGH the paged pool: writes the new
        token's k/v into its block and runs the split-S flash-decode HIP
        kernel over the block table — the padded [n, Hkv, L, D] views are
        never materialized (reference blocked_flash path). q/k/v are
        [n, 1, H(kv), D] (BSHD step slices); returns [n, 1, H, D] or None
        when ineligible (caller falls back to update() + SDPA)."""
        from ..ops.paged_attention import (paged_decode_attention,
                                           paged_decode_available)
        if self._q_len != 1 or not q.is_cuda or q.dtype != torch.bfloat16:
            return None
        kp = self.k[layer_idx]
        if not paged_decode_available(q.reshape(q.size(0), -1, q.size(-1)),
                                      kp):
            return None
        bs = self.block_size
        for i, s_ in enumerate(self._slots):
            p = int(self._starts[i])
            blk = self.block_table[s_][p // bs]
            self.k[layer_idx][blk, :, p % bs] = k[i, 0]
            self.v[layer_idx][blk, :, p % bs] = v[i, 0]
        nblk = (int(self._starts.max()) + 1 + bs - 1) // bs
        table = torch.tensor(
            [(self.block_table[s_] + [0] * nblk)[:nblk]
             for s_ in self._slots], dtype=torch.int32, device=q.device)
        lens = (self._starts + 1).to(q.device, torch.int32)
        o = paged_decode_attention(q[:, 0], kp, self.v[layer_idx], table,
                                   lens, scale=scale)
        return o.unsqueeze(1)

    def end_step(self):
        idx = torch.as_tensor(self._slots, device=self.lens.device)
        if self._packed:
            self.lens.index_add_(0, idx, torch.ones_like(idx))
        else:
            self.lens[idx] += self._q_len
        self._slots = None
        self.last_mask = None
