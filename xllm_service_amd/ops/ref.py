"""Pure-PyTorch fp32 reference implementations of every HIP op.

These serve two purposes:
  * numerics oracles for the GPU kernels (tests/test_gpu_ops.py compares the
    HIP kernels against these at fp32)
  * the CPU execution path (OPT-125m control-plane config)

They are intentionally simple and readable, not fast.
"""
from __future__ import annotations

import torch


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    return (xf * torch.rsqrt(var + eps) * w.float()).to(x.dtype)


def fused_add_rmsnorm(x, residual, w, eps):
    """Returns (normed, new_residual)."""
    summed = (x.float() + residual.float())
    out = rmsnorm(summed, w, eps).to(x.dtype)
    return out, summed.to(residual.dtype)


def rope_table(rot_dim: int, max_pos: int, base: float = 10000.0,
               scaling: float = 1.0) -> torch.Tensor:
    """cos/sin table [max_pos, rot_dim]: first half cos, second half sin."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rot_dim, 2).float() / rot_dim))
    t = torch.arange(max_pos).float() / scaling
    freqs = torch.outer(t, inv_freq)  # [max_pos, rot_dim/2]
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1)


def rope(positions, q, k, cos_sin, head_dim, rot_dim, mrope_sections=None):
    """NeoX rotate-half RoPE, applied out-of-place (reference). With
    mrope_sections (t, h, w summing to rot_dim//2) positions is [3, T] and
    frequency i takes its position from the section containing i."""
    def _apply(x):
        if mrope_sections:
            pos3 = positions
            T = pos3.shape[1]
            half = rot_dim // 2
            sec = torch.empty(half, dtype=torch.long)
            s0, s1, _ = mrope_sections
            sec[:s0] = 0
            sec[s0:s0 + s1] = 1
            sec[s0 + s1:] = 2
            # per (token, freq) position -> gather cos/sin rows
            pf = pos3[sec, :].T                      # [T, half]
            cos_t = cos_sin[:, :half][pf, torch.arange(half)]   # [T, half]
            sin_t = cos_sin[:, half:rot_dim][pf, torch.arange(half)]
            xs = x.reshape(T, -1, head_dim).float()
            cos = cos_t.unsqueeze(1)
            sin = sin_t.unsqueeze(1)
            x1 = xs[..., :half]
            x2 = xs[..., half:rot_dim]
            o1 = x1 * cos - x2 * sin
            o2 = x2 * cos + x1 * sin
            out = torch.cat([o1, o2, xs[..., rot_dim:]], dim=-1)
            return out.to(x.dtype).reshape(x.shape)
        T = positions.shape[0]
        xs = x.reshape(T, -1, head_dim).float()
        cs = cos_sin[positions]  # [T, rot_dim]
        cos = cs[:, : rot_dim // 2].unsqueeze(1)
        sin = cs[:, rot_dim // 2:].unsqueeze(1)
        x1 = xs[..., : rot_dim // 2]
        x2 = xs[..., rot_dim // 2: rot_dim]
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        out = torch.cat([o1, o2, xs[..., rot_dim:]], dim=-1)
        return out.to(x.dtype).reshape(x.shape)
    return _apply(q), _apply(k)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    g = x[..., :d].float()
    return (torch.nn.functional.silu(g) * x[..., d:].float()).to(x.dtype)


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    g = x[..., :d].float()
    return (torch.nn.functional.gelu(g, approximate="tanh") * x[..., d:].float()).to(x.dtype)


def reshape_and_cache(k, v, k_cache, v_cache, slot_mapping):
    """k/v: [T, n_kv, D]; caches [blocks, n_kv, bs, D]."""
    bs = k_cache.shape[2]
    for t in range(k.shape[0]):
        slot = int(slot_mapping[t])
        if slot < 0:
            continue
        b, off = divmod(slot, bs)
        k_cache[b, :, off, :] = k[t]
        v_cache[b, :, off, :] = v[t]


def gather_kv(seq_len, block_table, k_cache, v_cache):
    """Return contiguous K/V [seq_len, n_kv, D] for one sequence."""
    bs = k_cache.shape[2]
    nblk = (seq_len + bs - 1) // bs
    ks, vs = [], []
    for i in range(nblk):
        blk = int(block_table[i])
        take = min(bs, seq_len - i * bs)
        ks.append(k_cache[blk, :, :take, :].transpose(0, 1))
        vs.append(v_cache[blk, :, :take, :].transpose(0, 1))
    return torch.cat(ks, dim=0), torch.cat(vs, dim=0)


def paged_attn_decode(q, k_cache, v_cache, block_tables, seq_lens, scale):
    """q: [S, Hq, D] -> out [S, Hq, D]."""
    S, Hq, D = q.shape
    n_kv = k_cache.shape[1]
    G = Hq // n_kv
    out = torch.empty_like(q)
    for s in range(S):
        L = int(seq_lens[s])
        K, V = gather_kv(L, block_tables[s], k_cache, v_cache)  # [L, n_kv, D]
        for h in range(Hq):
            kv = h // G
            attn = (q[s, h].float() @ K[:, kv].float().T) * scale  # [L]
            p = torch.softmax(attn, dim=-1)
            out[s, h] = (p @ V[:, kv].float()).to(q.dtype)
    return out


def paged_attn_prefill(q, k_cache, v_cache, block_tables, cu_q, seq_lens, scale):
    """Varlen causal prefill over the paged cache.

    q: [total_q, Hq, D]; seq i has queries cu_q[i]:cu_q[i+1] and seq_lens[i]
    total keys (ctx = seq_lens[i] - q_len keys precede the new chunk).
    """
    total_q, Hq, D = q.shape
    n_kv = k_cache.shape[1]
    G = Hq // n_kv
    out = torch.empty_like(q)
    nseq = len(seq_lens)
    for s in range(nseq):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        qlen = q1 - q0
        L = int(seq_lens[s])
        ctx = L - qlen
        K, V = gather_kv(L, block_tables[s], k_cache, v_cache)
        for h in range(Hq):
            kv = h // G
            attn = (q[q0:q1, h].float() @ K[:, kv].float().T) * scale  # [qlen, L]
            # causal: query local i (global ctx+i) sees keys <= ctx+i
            dev = attn.device
            mask = torch.arange(L, device=dev)[None, :] > \
                (ctx + torch.arange(qlen, device=dev))[:, None]
            attn.masked_fill_(mask, float("-inf"))
            p = torch.softmax(attn, dim=-1)
            out[q0:q1, h] = (p @ V[:, kv].float()).to(q.dtype)
    return out


def greedy_sample(logits: torch.Tensor) -> torch.Tensor:
    return logits.float().argmax(dim=-1)


# ---------------------------------------------------------------------------
# Hybrid sequence-mixer ops (latent attention, decayed linear attention,
# grouped norms, gated residuals, routed experts). fp32 throughout.
# ---------------------------------------------------------------------------
def group_rmsnorm(x, w, eps, groups, out_dtype=None):
    """RMS norm over `groups` equal consecutive parts of the last dim."""
    sh = x.shape
    xg = x.float().reshape(*sh[:-1], groups, sh[-1] // groups)
    xg = xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)
    return (xg.reshape(sh) * w.float()).to(out_dtype or x.dtype)


def gated_norm_residual(res, y, gate, gate_bias, w, ls, mult, eps, groups):
    """res += mult * ls * group_rmsnorm(y * sigmoid(gate + gate_bias)) * w
    (res fp32, updated in place)."""
    g = gate.float()
    if gate_bias is not None:
        g = g + gate_bias.float()
    z = y.float() * torch.sigmoid(g)
    z = group_rmsnorm(z, w, eps, groups, torch.float32)
    res.add_(z * ls.float(), alpha=mult)
    return res


def norm_sigmoid_gate(o, w, gate, eps, out_dtype):
    """rmsnorm(o) * w * sigmoid(gate); w None skips the norm."""
    z = o.float()
    if w is not None:
        z = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return (z * torch.sigmoid(gate.float())).to(out_dtype)


def rope_interleaved(x, positions, inv_freq, mscale, rot_dims):
    """Rotate pairs (2i, 2i+1) of the first rot_dims entries of the last
    dim of x [T, H, D] by angle pos * inv_freq[i]; cos/sin scaled by mscale.
    Angles in fp64. Returns a new tensor."""
    a = positions.double()[:, None] * inv_freq.double()[None, :]
    cos = (torch.cos(a) * mscale).float()[:, None, :]
    sin = (torch.sin(a) * mscale).float()[:, None, :]
    xf = x.float()
    pr = xf[..., :rot_dims].reshape(*x.shape[:-1], rot_dims // 2, 2)
    u, v = pr[..., 0], pr[..., 1]
    rot = torch.stack([u * cos - v * sin, v * cos + u * sin], -1)
    out = torch.cat([rot.reshape(*x.shape[:-1], rot_dims),
                     xf[..., rot_dims:]], -1)
    return out.to(x.dtype)


def latent_kv_store(dkv, norm_w, eps, positions, inv_freq, mscale, rot_dims,
                    cache, slot_mapping, kv_rank):
    """cache row = [rmsnorm(dkv[:kv_rank]) * w | rope(dkv[kv_rank:])];
    cache [blocks, bs, kv_rank + rot]."""
    c = group_rmsnorm(dkv[:, :kv_rank], norm_w, eps, 1, torch.float32)
    kr = rope_interleaved(dkv[:, None, kv_rank:].float(), positions, inv_freq,
                          mscale, rot_dims)[:, 0]
    row = torch.cat([c, kr], -1).to(cache.dtype)
    bs = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1])
    ok = slot_mapping >= 0
    flat[slot_mapping[ok]] = row[ok]
    assert bs == cache.shape[1]


def _gather_latent(cache, table, L):
    bs = cache.shape[1]
    nblk = (L + bs - 1) // bs
    idx = table[:nblk].long()
    return cache[idx].reshape(nblk * bs, -1)[:L].float()


def latent_attn(q, cache, block_tables, cu_q, seq_lens, scale, kv_rank):
    """Causal softmax attention of per-head queries [T, H, W] against the
    shared latent rows [W] of the paged cache; values are the first kv_rank
    entries of each row. Sequence s has queries cu_q[s]:cu_q[s+1], the last
    of which sits at position seq_lens[s]-1. Returns fp32 [T, H, kv_rank]."""
    T, H, W = q.shape
    out = torch.zeros(T, H, kv_rank, dtype=torch.float32, device=q.device)
    for s in range(len(seq_lens)):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        L = int(seq_lens[s])
        ctx = L - (q1 - q0)
        kv = _gather_latent(cache, block_tables[s], L)          # [L, W]
        sc = torch.einsum("thw,lw->thl", q[q0:q1].float(), kv) * scale
        mask = torch.arange(L)[None, :] > (ctx + torch.arange(q1 - q0))[:, None]
        sc = sc.masked_fill(mask[:, None, :], float("-inf"))
        p = torch.softmax(sc, -1)
        out[q0:q1] = torch.einsum("thl,lr->thr", p, kv[:, :kv_rank])
    return out


def decay_linear_attn(q, k, v, decay, state, slots, cu_q, ctx_lens):
    """Per head S_t = decay * S_{t-1} + k_t v_t^T, o_t = S_t^T q_t with
    q = silu(q), k = silu(k), v = silu(v). state [slots, H, D, Dv] fp32 is
    read (unless ctx_len == 0: zero start) and written back per sequence;
    slot < 0 runs from zero and stores nothing. Returns fp32 [T, H, Dv]."""
    silu = torch.nn.functional.silu
    T, H, D = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=torch.float32, device=q.device)
    dec = decay.float()[:, None, None]
    for s in range(len(ctx_lens)):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        slot = int(slots[s])
        if slot >= 0 and int(ctx_lens[s]) > 0:
            S = state[slot].clone()
        else:
            S = torch.zeros(H, D, v.shape[-1], dtype=torch.float32)
        qs, ks, vs = (silu(a[q0:q1].float()).to(a.dtype).float()
                      for a in (q, k, v))
        for t in range(q1 - q0):
            S = dec * S + ks[t][:, :, None] * vs[t][:, None, :]
            out[q0 + t] = torch.einsum("hdv,hd->hv", S, qs[t])
        if slot >= 0:
            state[slot] = S
    return out


def moe_route(h, w_router, top, n_groups, keep):
    """Sigmoid-scored top-k routing with group limiting: experts form
    n_groups equal neighbouring groups scored by the sum of their two
    largest scores; only the best `keep` groups are eligible. Returns
    (ids [T, top] int32, weights [T, top] fp32 = raw scores)."""
    z = h.float() @ w_router.float().T
    s = torch.sigmoid(z)
    T, E = s.shape
    sm = s
    if n_groups > 1:
        sg = s.view(T, n_groups, E // n_groups)
        gs = sg.topk(min(2, E // n_groups), -1).values.sum(-1)
        best = gs.topk(keep, -1).indices
        gm = torch.zeros_like(gs, dtype=torch.bool).scatter(1, best, True)
        sm = sg.masked_fill(~gm[:, :, None], float("-inf")).reshape(T, E)
    idx = sm.topk(top, -1).indices
    return idx.to(torch.int32), s.gather(1, idx)


def silu_mul(x):
    """[..., 2F] -> silu(x[..., :F]) * x[..., F:], dtype preserved."""
    return silu_and_mul(x)
