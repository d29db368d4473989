"""Routed-expert feed-forward.

Router: fp32 logits, sigmoid scores, optional group limiting (experts form
equal neighbouring groups, a group scores the sum of its two best experts,
only the best `keep` groups are eligible), top-k, weights = raw scores.
Experts: down(silu(gate h) * (up h)), no biases; gate and up are one merged
matrix per expert.

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
                 n_groups: int, keep: int, dtype, dense_max_tokens: int = 64):
        super().__init__()
        if experts % n_groups or keep > n_groups or \
                keep * (experts // n_groups) < top:
            raise ValueError("inconsistent routing constants")
        self.width, self.ff, self.experts, self.top = width, ff, experts, top
        self.n_groups, self.keep = n_groups, keep
        self.dense_max_tokens = dense_max_tokens
        self.router = nn.Parameter(torch.empty(experts, width,
                                               dtype=torch.float32))
        self.w_gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width,
                                                  dtype=dtype))
        self.w_down = nn.Parameter(torch.empty(experts, width, ff,
                                               dtype=dtype))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """h [T, width] (model dtype) -> fp32 [T, width]."""
        T = h.shape[0]
        ids, wts = hops.moe_route(h, self.router, self.top, self.n_groups,
                                  self.keep)
        capturing = h.is_cuda and torch.cuda.is_current_stream_capturing()
        if T <= self.dense_max_tokens or capturing:
            gu = torch.matmul(h, self.w_gate_up.transpose(1, 2))  # [E,T,2ff]
            act = hops.silu_mul(gu)
            y = torch.bmm(act, self.w_down.transpose(1, 2))       # [E,T,W]
            rows = ids * T + torch.arange(T, dtype=torch.int32,
                                          device=h.device)[:, None]
            return hops.moe_combine(y, rows, wts, T)
        flat = ids.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        counts_t = torch.bincount(flat, minlength=self.experts)
        counts = counts_t.tolist()                 # the one host round trip
        cap, total = max(counts), T * self.top
        if cap * self.experts <= 1.5 * total + 16 * self.experts:
            # near-even load: pad every expert to `cap` rows and run all of
            # them as two batched GEMMs
            e_sorted = flat[order]
            starts = torch.cumsum(counts_t, 0) - counts_t
            dest = e_sorted * cap + (torch.arange(total, device=h.device)
                                     - starts[e_sorted])
            xs = h.new_zeros(self.experts * cap, self.width)
            xs[dest] = h[order // self.top]
            gu = torch.bmm(xs.view(self.experts, cap, self.width),
                           self.w_gate_up.transpose(1, 2))
            y = torch.bmm(hops.silu_mul(gu), self.w_down.transpose(1, 2))
            rows = torch.empty_like(dest)
            rows[order] = dest
            return hops.moe_combine(y.view(-1, self.width),
                                    rows.view(T, self.top).to(torch.int32),
                                    wts, T)
        xs = h[order // self.top]
        ys = torch.empty(T * self.top, self.width, dtype=h.dtype,
                         device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                seg = slice(at, at + n)
                act = hops.silu_mul(F.linear(xs[seg], self.w_gate_up[e]))
                ys[seg] = F.linear(act, self.w_down[e])
                at += n
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=h.device)
        rows = inv.view(T, self.top).to(torch.int32)
        return hops.moe_combine(ys, rows, wts, T)
