"""Sequence mixers beyond plain multi-head attention.

LatentAttention        softmax attention whose keys and values are linear
                       images of one cached low-rank latent per token, plus
                       one rotated key part shared by all heads. Queries are
                       folded through the key up-projection so the kernel
                       works on the cached rows directly; the value
                       up-projection follows the weighted sum.
DecayLinearAttention   per-head state S <- decay * S + k v^T, o = S^T q with
                       SiLU feature maps; the state lives in a slot pool.

Both take the slice of a merged input projection that belongs to them and
return the mixer output in the model dtype. Sizes and constants are
constructor arguments.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.engine.cache_spec import (PagedLatent, RecurrentState,
                                                SharedCache)
from xllm_service_amd.engine.metadata import AttnMetadata
from xllm_service_amd.ops import hybrid as hops


def scaled_rope_frequencies(rot: dict):
    """Per-pair inverse frequencies (fp64) and the cos/sin multiplier of a
    rotary config {base, dims, scaling?}. With `scaling` = {factor, original,
    fast, slow} the frequencies are blended between f_i and f_i / factor by
    a linear ramp over the pair index between the pairs that complete `fast`
    and `slow` turns within `original` positions (YaRN), and cos/sin are
    multiplied by 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])

    def pair_at(turns):
        return (dims * math.log(float(sc["original"]) /
                                (2.0 * math.pi * float(turns)))
                / (2.0 * math.log(base)))
    lo = max(math.floor(pair_at(sc["fast"])), 0)
    hi = min(math.ceil(pair_at(sc["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


class LatentAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, rot_dim: int,
                 vdim: int, kv_rank: int, scale: float, rot: dict,
                 norm_eps: float, kv_from: Optional[int], dtype):
        super().__init__()
        self.heads, self.dim, self.rot_dim = heads, dim, rot_dim
        self.vdim, self.kv_rank = vdim, kv_rank
        self.scale, self.eps, self.kv_from = float(scale), norm_eps, kv_from
        self.rot_dims = int(rot["dims"])
        if self.rot_dims > rot_dim or self.rot_dims % 2:
            raise ValueError("rotary dims must be even and <= rot_dim")
        inv_freq, self.mscale = scaled_rope_frequencies(rot)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        self.q_width = heads * (dim + rot_dim)
        self.dkv_width = 0 if kv_from is not None else kv_rank + rot_dim
        self.g_width = heads * vdim
        # merged-projection rows owned by this mixer: [q | dkv | g]
        self.in_width = self.q_width + self.dkv_width + self.g_width
        if kv_from is None:
            self.dkv_norm = nn.Parameter(torch.ones(kv_rank,
                                                    dtype=torch.float32))
        # key up-projection per head [H, dim, r]; value up-projection
        # transposed per head [H, r, vdim]
        self.w_uk = nn.Parameter(torch.empty(heads, dim, kv_rank, dtype=dtype))
        self.w_uv_t = nn.Parameter(torch.empty(heads, kv_rank, vdim,
                                               dtype=dtype))
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim,
                                               dtype=dtype))

    def cache_spec(self):
        if self.kv_from is not None:
            return SharedCache(self.kv_from)
        return PagedLatent(self.kv_rank + self.rot_dim)

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        T = proj.shape[0]
        H, dim, rd, r = self.heads, self.dim, self.rot_dim, self.kv_rank
        q = proj[:, :self.q_width].unflatten(-1, (H, dim + rd))
        hops.rope_interleaved_(q, positions, self.inv_freq, self.mscale, dim,
                               self.rot_dims)
        if self.kv_from is None:
            dkv = proj[:, self.q_width:self.q_width + self.dkv_width]
            hops.latent_kv_store(dkv, self.dkv_norm, self.eps, positions,
                                 self.inv_freq, self.mscale, self.rot_dims,
                                 cache, meta.slot_mapping, r)
        gate = proj[:, self.q_width + self.dkv_width:self.in_width]
        # fold the queries through the key up-projection: [H,T,dim]x[H,dim,r]
        q_abs = torch.bmm(q[..., :dim].transpose(0, 1), self.w_uk)
        qf = torch.empty(T, H, r + rd, dtype=proj.dtype, device=proj.device)
        qf[..., :r] = q_abs.transpose(0, 1)
        qf[..., r:] = q[..., dim:]
        lat = torch.empty(T, H, r, dtype=torch.float32, device=proj.device)
        np_, nd = meta.num_prefill_tokens, meta.num_decode_tokens
        if np_:
            hops.latent_attn(qf[:np_], cache, meta.prefill_block_tables,
                             meta.cu_q, meta.prefill_seq_lens, self.scale, r,
                             lat[:np_])
        if nd:
            hops.latent_attn(qf[np_:], cache, meta.decode_block_tables, None,
                             meta.decode_seq_lens, self.scale, r, lat[np_:])
        # value up-projection per head: [H,T,r] x [H,r,vdim]
        o = torch.bmm(lat.to(proj.dtype).transpose(0, 1), self.w_uv_t)
        o = o.transpose(0, 1).reshape(T, H * self.vdim)
        y = hops.norm_sigmoid_gate(o.float(), None, gate, self.eps, proj.dtype)
        return F.linear(y, self.o_proj)


class DecayLinearAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay,
                 norm_eps: float, dtype):
        super().__init__()
        if len(decay) != heads:
            raise ValueError("one decay per head")
        self.heads, self.dim, self.vdim, self.eps = heads, dim, vdim, norm_eps
        self.register_buffer("decay", torch.tensor(decay, dtype=torch.float32),
                             persistent=False)
        self.qk_width = heads * dim
        self.v_width = heads * vdim
        # merged-projection rows owned by this mixer: [q | k | v | g]
        self.in_width = 2 * self.qk_width + 2 * self.v_width
        self.out_norm = nn.Parameter(torch.ones(self.v_width,
                                                dtype=torch.float32))
        self.o_proj = nn.Parameter(torch.empty(width, self.v_width,
                                               dtype=dtype))

    def cache_spec(self):
        return RecurrentState(self.heads, self.dim, self.vdim)

    def forward(self, proj, positions, state, meta: AttnMetadata, aux):
        T = proj.shape[0]
        a, b = self.qk_width, self.v_width
        q, k = proj[:, :a], proj[:, a:2 * a]
        v, gate = proj[:, 2 * a:2 * a + b], proj[:, 2 * a + b:self.in_width]
        o = torch.empty(T, self.heads, self.vdim, dtype=torch.float32,
                        device=proj.device)
        np_, nd = meta.num_prefill_tokens, meta.num_decode_tokens
        if np_:
            hops.decay_attn(q[:np_], k[:np_], v[:np_], self.decay, state,
                            meta.prefill_state_slots, meta.cu_q,
                            meta.prefill_ctx_lens, o[:np_],
                            max_q_len=meta.max_prefill_len)
        if nd:
            hops.decay_attn(q[np_:], k[np_:], v[np_:], self.decay, state,
                            meta.decode_state_slots, None,
                            aux["decode_ctx_lens"], o[np_:])
        y = hops.norm_sigmoid_gate(o.view(T, b), self.out_norm, gate,
                                   self.eps, proj.dtype)
        return F.linear(y, self.o_proj)
