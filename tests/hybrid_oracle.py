"""Slow, plain fp64 oracle for the hybrid decoder (Pugovik) — one function
per mechanism, written from the equations, sharing nothing with the package:

  grouped RMS norm      y = x / sqrt(mean_g(x^2) + eps) * w   per group g
  rotary (pairs)        (u, v) -> (u c - v s, v c + u s), angle p * f_i,
                        f_i blended by a YaRN ramp, c/s scaled
  latent attention      c = rms(W_dkv h)[:r], shared rotated key tail;
                        k_h = W_uk c, v_h = W_uv c, causal softmax, sigmoid
                        output gate, output projection
  decayed linear attn   S = a_h S + k v^T, o = S^T q, silu feature maps,
                        rms + sigmoid gate on the concatenated heads
  routed experts        sigmoid scores, group-limited top-k, raw-score mix
  block                 x += m * ls * gnorm(sub(gnorm(x)) * sigmoid(W h + b))

Also a checkpoint generator and a minimal safetensors writer so tests can
hand the engine a model folder of their own making.
"""
import json
import math
import os
import struct

import numpy as np
import torch

F64 = torch.float64


# ---------------------------------------------------------------- mechanisms
def o_gnorm(x, w, eps, groups):
    out = torch.empty_like(x)
    n = x.shape[-1] // groups
    for g in range(groups):
        part = x[..., g * n:(g + 1) * n]
        out[..., g * n:(g + 1) * n] = part / torch.sqrt(
            (part ** 2).mean(-1, keepdim=True) + eps)
    return out * w


def o_freqs(rot):
    dims, base = rot["dims"], rot["base"]
    fs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return fs, 1.0
    def where(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (
            2 * math.log(base))
    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    out = []
    for i, f in enumerate(fs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / sc["factor"] * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def o_rotate(vec, pos, rot):
    """vec: 1-D fp64; rotates its first rot['dims'] entries pairwise."""
    fs, mult = o_freqs(rot)
    out = vec.clone()
    for i, f in enumerate(fs):
        a = pos * f
        c, s = math.cos(a) * mult, math.sin(a) * mult
        u, v = float(vec[2 * i]), float(vec[2 * i + 1])
        out[2 * i] = u * c - v * s
        out[2 * i + 1] = v * c + u * s
    return out


def o_latent_attention(Wt, p, mc, h, eps, latents, li):
    T = h.shape[0]
    H, d, rd, vd, r = (mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"],
                       mc["kv_rank"])
    q = h @ Wt[p + "q"].T
    if "kv_from" in mc:
        c, kr = latents[mc["kv_from"]]
    else:
        dkv = h @ Wt[p + "dkv"].T
        c = o_gnorm(dkv[:, :r], Wt[p + "dkv.norm"], eps, 1)
        kr = torch.stack([o_rotate(dkv[t, r:], t, mc["rot"])
                          for t in range(T)])
        latents[li] = (c, kr)
    heads_out = []
    for hh in range(H):
        qh = q[:, hh * (d + rd):(hh + 1) * (d + rd)]
        qn = qh[:, :d]
        qr = torch.stack([o_rotate(qh[t, d:], t, mc["rot"])
                          for t in range(T)])
        k = c @ Wt[p + "uk"][hh * d:(hh + 1) * d].T
        v = c @ Wt[p + "uv"][hh * vd:(hh + 1) * vd].T
        o = torch.zeros(T, vd, dtype=F64)
        for t in range(T):
            s = (k[:t + 1] @ qn[t] + kr[:t + 1] @ qr[t]) * mc["scale"]
            w = torch.softmax(s, 0)
            o[t] = w @ v[:t + 1]
        heads_out.append(o)
    o = torch.cat(heads_out, -1) * torch.sigmoid(h @ Wt[p + "g"].T)
    return o @ Wt[p + "o"].T


def o_decay_attention(Wt, p, mc, h, eps):
    T = h.shape[0]
    H, d, vd = mc["heads"], mc["dim"], mc["vdim"]
    silu = lambda z: z * torch.sigmoid(z)
    q, k, v = (silu(h @ Wt[p + n].T) for n in "qkv")
    o = torch.zeros(T, H * vd, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, vd, dtype=F64)
        for t in range(T):
            kt = k[t, hh * d:(hh + 1) * d]
            vt = v[t, hh * vd:(hh + 1) * vd]
            S = mc["decay"][hh] * S + torch.outer(kt, vt)
            o[t, hh * vd:(hh + 1) * vd] = S.T @ q[t, hh * d:(hh + 1) * d]
    o = o_gnorm(o, Wt[p + "norm"], eps, 1) * torch.sigmoid(h @ Wt[p + "g"].T)
    return o @ Wt[p + "o"].T


def o_route(scores, rc):
    """scores: list of floats; returns chosen expert indices."""
    E, top = rc["experts"], rc["top"]
    ok = list(range(E))
    g = rc.get("groups")
    if g and g["count"] > 1:
        n = E // g["count"]
        gscore = []
        for gi in range(g["count"]):
            best = sorted(scores[gi * n:(gi + 1) * n], reverse=True)[:2]
            gscore.append(sum(best))
        keep = sorted(range(g["count"]), key=lambda i: -gscore[i])[:g["keep"]]
        ok = [e for e in range(E) if e // n in keep]
    return sorted(ok, key=lambda e: -scores[e])[:top]


def o_experts(Wt, p, fc, h):
    silu = lambda z: z * torch.sigmoid(z)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        s = torch.sigmoid(Wt[p + "router"] @ h[t])
        for e in o_route(s.tolist(), fc["router"]):
            pe = f"{p}e{e}."
            mid = silu(Wt[pe + "gate"] @ h[t]) * (Wt[pe + "up"] @ h[t])
            out[t] += s[e] * (Wt[pe + "down"] @ mid)
    return out


def o_forward(cfg, Wt, tokens):
    """Returns (logits [T, vocab], residual stream after every layer)."""
    eps, G, m = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"]
    x = o_gnorm(Wt["embed"][torch.tensor(tokens)], Wt["embed.norm"], eps, G)
    latents, trail = {}, []
    for li, L in enumerate(cfg["layers"]):
        p = f"l{li}."
        h = o_gnorm(x, Wt[p + "norm1"], eps, G)
        if L["type"] == "latent_attention":
            y = o_latent_attention(Wt, p + "mix.", L["mixer"], h, eps,
                                   latents, li)
        else:
            y = o_decay_attention(Wt, p + "mix.", L["mixer"], h, eps)
        y = y * torch.sigmoid(h @ Wt[p + "rg1"].T + Wt[p + "rg1.b"])
        x = x + m * Wt[p + "ls1"] * o_gnorm(y, Wt[p + "norm1b"], eps, G)
        if L.get("mlp"):
            h = o_gnorm(x, Wt[p + "norm2"], eps, G)
            y = o_experts(Wt, p + "mlp.", L["mlp"], h)
            y = y * torch.sigmoid(h @ Wt[p + "rg2"].T + Wt[p + "rg2.b"])
            x = x + m * Wt[p + "ls2"] * o_gnorm(y, Wt[p + "norm2b"], eps, G)
        trail.append(x.clone())
    x = o_gnorm(x, Wt["final.norm"], eps, G)
    return x @ Wt["head"].T, trail


# ------------------------------------------------------- checkpoints for tests
def make_config(width=48, vocab=96, groups=3, mult=0.4, eps=1e-5, layers=None):
    return dict(architecture="Pugovik", vocab=vocab, width=width,
                norm=dict(eps=eps, groups=groups), residual_mult=mult,
                layers=layers)


def lin_layer(heads=3, dim=8, vdim=12, decay=None, mlp=None):
    decay = decay or [0.5 + 0.45 * i / max(heads - 1, 1) for i in range(heads)]
    return dict(type="lightning", mlp=mlp,
                mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=decay))


def lat_layer(heads=2, dim=12, rot_dim=8, vdim=10, kv_rank=24, dims=None,
              scaling=True, kv_from=None, mlp=None, base=10000.0):
    rot = dict(base=base, dims=dims or rot_dim)
    if scaling:
        rot["scaling"] = dict(factor=3.0, original=64, fast=8.0, slow=1.0)
    mixer = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                 kv_rank=kv_rank, scale=(dim + rot_dim) ** -0.5, rot=rot)
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return dict(type="latent_attention", mixer=mixer, mlp=mlp)


def moe(experts=6, top=2, ff=16, count=3, keep=2):
    r = dict(experts=experts, top=top)
    if count:
        r["groups"] = dict(count=count, keep=keep)
    return dict(kind="moe", expert=dict(ff=ff), router=r)


def make_weights(cfg, seed=0, spread_router=True):
    """Random checkpoint (values exactly representable in bf16)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    out = {}

    def mat(name, rows, cols, std=None):
        std = std if std is not None else 1.2 / math.sqrt(cols)
        out[name] = (torch.randn(rows, cols, generator=g) * std)

    def vec(name, n, center=1.0, spread=0.3):
        out[name] = center + spread * (torch.rand(n, generator=g) * 2 - 1)

    mat("embed", cfg["vocab"], W, 1.0)
    vec("embed.norm", W)
    vec("final.norm", W)
    mat("head", cfg["vocab"], W)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        for n in ("norm1", "norm1b"):
            vec(p + n, W)
        vec(p + "ls1", W, 0.8, 0.4)
        mat(p + "rg1", W, W)
        vec(p + "rg1.b", W, 0.0, 0.5)
        if L["type"] == "lightning":
            H, d, vd = m["heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * d, W)
            mat(p + "mix.k", H * d, W)
            mat(p + "mix.v", H * vd, W)
            mat(p + "mix.g", H * vd, W)
            mat(p + "mix.o", W, H * vd)
            vec(p + "mix.norm", H * vd)
        else:
            H, d, rd, vd, r = (m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                               m["kv_rank"])
            mat(p + "mix.q", H * (d + rd), W, 2.0 / math.sqrt(W))
            if "kv_from" not in m:
                mat(p + "mix.dkv", r + rd, W, 2.0 / math.sqrt(W))
                vec(p + "mix.dkv.norm", r)
            mat(p + "mix.uk", H * d, r)
            mat(p + "mix.uv", H * vd, r)
            mat(p + "mix.g", H * vd, W)
            mat(p + "mix.o", W, H * vd)
        if L.get("mlp"):
            fc = L["mlp"]
            E, ff = fc["router"]["experts"], fc["expert"]["ff"]
            for n in ("norm2", "norm2b"):
                vec(p + n, W)
            vec(p + "ls2", W, 0.8, 0.4)
            mat(p + "rg2", W, W)
            vec(p + "rg2.b", W, 0.0, 0.5)
            # a wide router keeps expert scores apart (no near-ties)
            mat(p + "mlp.router", E, W, (3.0 if spread_router else 1.0)
                / math.sqrt(W))
            for e in range(E):
                mat(f"{p}mlp.e{e}.gate", ff, W)
                mat(f"{p}mlp.e{e}.up", ff, W)
                mat(f"{p}mlp.e{e}.down", W, ff)
    return {k: v.to(torch.bfloat16) for k, v in out.items()}


def write_safetensors(path, tensors):
    header, blobs, at = {}, [], 0
    for name, t in tensors.items():
        assert t.dtype == torch.bfloat16
        raw = t.contiguous().view(torch.int16).numpy().tobytes()
        header[name] = dict(dtype="BF16", shape=list(t.shape),
                            data_offsets=[at, at + len(raw)])
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


def write_model_dir(folder, cfg, weights):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return folder


def as_f64(weights):
    return {k: v.to(F64) for k, v in weights.items()}


def rel_err(got, want):
    """Per-row error: rms of the mean-free difference over the row's rms."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    ref = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() /
            ref.pow(2).mean(-1).sqrt().clamp_min(1e-12))
