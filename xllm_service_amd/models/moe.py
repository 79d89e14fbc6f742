"""Routed-expert feed-forward.

Router: fp32 logits, sigmoid scores, optional group limiting (experts form
equal neighbouring groups, a group scores the sum of its two best experts,
only the best `keep` groups are eligible), top-k, weights = raw scores.
Experts: down(silu(gate h) * (up h)), no biases; gate and up are one merged
matrix per expert.

Options: softmax scores over all experts, a correction added to the scores
for the choice only, groups scored by their best expert, weights divided by
their sum, `identity` further router outputs that stand for experts without
tensors whose output is their input, and a shared expert of the same form
that every token uses (added to the routed sum in fp32).

Two execution shapes over the same weights, both ending in the fp32 combine
kernel: few tokens (decode batches, graph capture) run every expert as one
batched GEMM over all tokens — at those sizes the step is bound by reading
the expert weights, which a token-sorted pass would read as well, and it
needs no host round trip; many tokens are sorted by expert and each expert
multiplies only its own rows (as one padded batched GEMM when the load is
near-even, expert by expert otherwise).
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.ops import hybrid as hops


class RoutedExperts(nn.Module):
    def __init__(self, width: int, ff: int, experts: int, top: int,
                 n_groups: int, keep: int, dtype, dense_max_tokens: int = 64,
                 *, identity: int = 0, softmax: bool = False,
                 correction: bool = False, group_max: bool = False,
                 normalize: bool = False, shared_ff: int = 0):
        super().__init__()
        n_all = experts + identity
        if n_all % n_groups or keep > n_groups or \
                keep * (n_all // n_groups) < top:
            raise ValueError("inconsistent routing constants")
        self.width, self.ff, self.experts, self.top = width, ff, experts, top
        self.n_groups, self.keep = n_groups, keep
        self.identity, self.softmax = identity, softmax
        self.group_max, self.normalize = group_max, normalize
        self.dense_max_tokens = dense_max_tokens
        self.router = nn.Parameter(torch.empty(n_all, width,
                                               dtype=torch.float32))
        self.correction = nn.Parameter(torch.zeros(
            n_all, dtype=torch.float32)) if correction else None
        self.w_gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width,
                                                  dtype=dtype))
        self.w_down = nn.Parameter(torch.empty(experts, width, ff,
                                               dtype=dtype))
        self.shared_ff = shared_ff
        if shared_ff:
            self.shared_gate_up = nn.Parameter(torch.empty(
                2 * shared_ff, width, dtype=dtype))
            self.shared_down = nn.Parameter(torch.empty(width, shared_ff,
                                                        dtype=dtype))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """h [T, width] (model dtype) -> fp32 [T, width]."""
        T, E = h.shape[0], self.experts
        ids, wts = hops.moe_route(
            h, self.router, self.top, self.n_groups, self.keep,
            softmax=self.softmax, correction=self.correction,
            group_max=self.group_max, normalize=self.normalize)
        extra = None
        if self.shared_ff:
            extra = F.linear(hops.silu_mul(F.linear(h, self.shared_gate_up)),
                             self.shared_down)
        ident = h if self.identity else None
        capturing = h.is_cuda and torch.cuda.is_current_stream_capturing()
        if T <= self.dense_max_tokens or capturing:
            gu = torch.matmul(h, self.w_gate_up.transpose(1, 2))  # [E,T,2ff]
            act = hops.silu_mul(gu)
            y = torch.bmm(act, self.w_down.transpose(1, 2))       # [E,T,W]
            rows = ids * T + torch.arange(T, dtype=torch.int32,
                                          device=h.device)[:, None]
            if self.identity:
                rows = torch.where(ids >= E, -1, rows)
            return hops.moe_combine(y, rows, wts, T, ident, extra)
        # identity choices sort behind every expert and take no rows
        flat = ids.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        counts_t = torch.bincount(flat, minlength=E + self.identity)
        counts = counts_t.tolist()                 # the one host round trip
        total = sum(counts[:E])                    # pairs that use an expert
        order = order[:total]
        counts_t, counts = counts_t[:E], counts[:E]
        cap = max(counts) if counts else 0
        rows = torch.full((T * self.top,), -1, dtype=torch.int32,
                          device=h.device)
        if total == 0:
            y = h.new_zeros(1, self.width)
            return hops.moe_combine(y, rows.view(T, self.top), wts, T, ident,
                                    extra)
        if cap * E <= 1.5 * total + 16 * E:
            # near-even load: pad every expert to `cap` rows and run all of
            # them as two batched GEMMs
            e_sorted = flat[order]
            starts = torch.cumsum(counts_t, 0) - counts_t
            dest = e_sorted * cap + (torch.arange(total, device=h.device)
                                     - starts[e_sorted])
            xs = h.new_zeros(E * cap, self.width)
            xs[dest] = h[order // self.top]
            gu = torch.bmm(xs.view(E, cap, self.width),
                           self.w_gate_up.transpose(1, 2))
            y = torch.bmm(hops.silu_mul(gu), self.w_down.transpose(1, 2))
            rows[order] = dest.to(torch.int32)
            return hops.moe_combine(y.view(-1, self.width),
                                    rows.view(T, self.top), wts, T, ident,
                                    extra)
        xs = h[order // self.top]
        ys = torch.empty(total, self.width, dtype=h.dtype, device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                seg = slice(at, at + n)
                act = hops.silu_mul(F.linear(xs[seg], self.w_gate_up[e]))
                ys[seg] = F.linear(act, self.w_down[e])
                at += n
        rows[order] = torch.arange(total, dtype=torch.int32, device=h.device)
        return hops.moe_combine(ys, rows.view(T, self.top), wts, T, ident,
                                extra)
