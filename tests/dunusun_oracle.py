"""Slow, plain fp64 oracle for the Dunusun decoder — one function per
mechanism, written from the equations, sharing nothing with the package.

  layer norm            (x - mean) / sqrt(var + eps) * w + b
  short convolution     y_t = sum_j w[:, j] u_(t - taps + 1 + j) (+ b), zeros
                        before the start of the sequence
  rotary (pairs)        (u, v) -> (u c - v s, v c + u s), angle p * f_i on
                        the first `dims` entries of a head
  selective state space S = exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x,
                        gated by silu(z), grouped RMS norm
  soft-capped attention convolved + rotated q/k, grouped key/value heads,
                        cap * tanh(score / cap), causal softmax, sigmoid gate
  gated linear attn     S = diag(alpha) S + k v^T, o = S^T q with
                        alpha = sigmoid(low-rank(h))^(1/tau); per-head RMS
                        norm, silu gate
  several residuals     u = sum_s in[s] x_s; x_t <- sum_s mix[s,t] x_s +
                        out[t] y
  looped layers         a run of layers repeated with the same weights

Also a checkpoint generator and a minimal safetensors writer so tests can
hand the engine a model folder of their own making.
"""
import json
import math
import os
import struct

import torch

F64 = torch.float64


# ---------------------------------------------------------------- mechanisms
def o_layernorm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def o_rms(x, eps):
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)


def o_silu(x):
    return x / (1.0 + torch.exp(-x))


def o_softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(
        x, max=30.0))))


def o_conv(u, w, b=None):
    """u [T, C], w [C, taps]: the last column multiplies the current row."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * u[src]
        if b is not None:
            out[t] += b
    return out


def o_rotate(vec, pos, rot):
    """vec 1-D: its first rot['dims'] entries are turned pair by pair."""
    out = vec.clone()
    dims, base = int(rot["dims"]), float(rot["base"])
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, v = float(vec[2 * i]), float(vec[2 * i + 1])
        out[2 * i] = u * c - v * s
        out[2 * i + 1] = v * c + u * s
    return out


def o_state_space(Wt, p, mc, h, eps):
    """h [T, W] -> [T, W]; the recurrence runs token by token."""
    H, P, N, G = mc["heads"], mc["vdim"], mc["state"], mc["groups"]
    inner = H * P
    T = h.shape[0]
    proj = h @ Wt[p + "in"].T
    z = proj[:, :inner]
    xbc = o_silu(o_conv(proj[:, inner:2 * inner + 2 * G * N],
                        Wt[p + "conv"], Wt[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = o_softplus(proj[:, 2 * inner + 2 * G * N:] + Wt[p + "dt_bias"])
    A = torch.exp(Wt[p + "A_log"])
    y = torch.zeros(T, H, P, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = math.exp(-float(A[hd]) * float(dt[t, hd])) * S \
                + float(dt[t, hd]) * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + Wt[p + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * o_silu(z)
    ng = mc["norm_groups"]
    n = inner // ng
    parts = [o_rms(y[:, i * n:(i + 1) * n], eps) for i in range(ng)]
    return (torch.cat(parts, -1) * Wt[p + "norm"]) @ Wt[p + "o"].T


def o_capped_attention(Wt, p, mc, h):
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q = o_conv(h @ Wt[p + "q"].T, Wt[p + "q.conv"]).reshape(T, H, D)
    k = o_conv(h @ Wt[p + "k"].T, Wt[p + "k.conv"]).reshape(T, G, D)
    v = o_conv(h @ Wt[p + "v"].T, Wt[p + "v.conv"]).reshape(T, G, Dv)
    rot = mc.get("rot")
    if rot:
        for t in range(T):
            for i in range(H):
                q[t, i] = o_rotate(q[t, i], t, rot)
            for i in range(G):
                k[t, i] = o_rotate(k[t, i], t, rot)
    cap = mc.get("softcap")
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            sc = (k[:t + 1, g] @ q[t, hd]) * mc["scale"]
            if cap:
                sc = cap * torch.tanh(sc / cap)
            wgt = torch.softmax(sc, 0)
            o[t, hd] = wgt @ v[:t + 1, g]
    gate = torch.sigmoid(h @ Wt[p + "g"].T)
    return (o.reshape(T, H * Dv) * gate) @ Wt[p + "o"].T


def o_gated_linear(Wt, p, mc, h, eps):
    H, D, Dv, tau = mc["heads"], mc["dim"], mc["vdim"], mc["tau"]
    T = h.shape[0]
    q = (h @ Wt[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ Wt[p + "k"].T).reshape(T, H, D)
    v = (h @ Wt[p + "v"].T).reshape(T, H, Dv)
    zz = (h @ Wt[p + "a1"].T) @ Wt[p + "a2"].T + Wt[p + "a2.b"]
    alpha = (torch.sigmoid(zz) ** (1.0 / tau)).reshape(T, H, D)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = alpha[t, hd][:, None] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = o_rms(o, eps) * Wt[p + "norm"]
    return (o.reshape(T, H * Dv) * o_silu(h @ Wt[p + "g"].T)) @ Wt[p + "o"].T


def o_mixer(Wt, p, lc, h, eps):
    mc = lc["mixer"]
    if lc["type"] == "mamba2":
        return o_state_space(Wt, p + "mix.", mc, h, eps)
    left = o_capped_attention(Wt, p + "mix.left.", mc["left"], h)
    right = o_gated_linear(Wt, p + "mix.right.", mc["right"], h, eps)
    return mc["left_scale"] * left + mc["right_scale"] * right


def o_ff(Wt, p, h):
    return (torch.relu(h @ Wt[p + "up"].T) ** 2) @ Wt[p + "down"].T


def o_layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    body = list(range(lp["start"], lp["stop"]))
    return list(range(lp["start"])) + body * lp["times"] \
        + list(range(lp["stop"], n))


def o_forward(cfg, Wt, tokens):
    """-> logits [T, vocab], residual after every layer run [runs, T, W]
    (the sum of the streams)."""
    eps = cfg["norm"]["eps"]
    s_n = cfg.get("streams")
    e = Wt["embed"][torch.tensor(tokens)]
    xs = [e.clone() for _ in range(s_n or 1)]
    after = []
    for li in o_layer_runs(cfg):
        lc, p = cfg["layers"][li], f"l{li}."
        subs = [(1, lambda u: o_mixer(Wt, p, lc, u, eps))]
        if lc.get("mlp") is not None:
            subs.append((2, lambda u: o_ff(Wt, p + "mlp.", u)))
        for qn, fn in subs:
            nw, nb = Wt[f"{p}norm{qn}"], Wt[f"{p}norm{qn}.b"]
            if s_n is None:
                xs = [xs[0] + fn(o_layernorm(xs[0], nw, nb, eps))]
                continue
            hin, hout = Wt[f"{p}hc{qn}.in"], Wt[f"{p}hc{qn}.out"]
            hmix = Wt[f"{p}hc{qn}.mix"]
            u = sum(hin[s] * xs[s] for s in range(s_n))
            y = fn(o_layernorm(u, nw, nb, eps))
            xs = [sum(hmix[s, t] * xs[s] for s in range(s_n)) + hout[t] * y
                  for t in range(s_n)]
        after.append(sum(xs))
    x = o_layernorm(sum(xs), Wt["final.norm"], Wt["final.norm.b"], eps)
    logits = x @ Wt["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(after)


# ------------------------------------------------------- configs and weights
def ssm_layer(heads=4, vdim=6, state=5, groups=2, norm_groups=2, conv=3,
              mlp=10):
    return {"type": "mamba2",
            "mixer": dict(heads=heads, vdim=vdim, state=state, groups=groups,
                          norm_groups=norm_groups, conv=conv),
            "mlp": None if mlp is None else dict(kind="dense", ff=mlp)}


def par_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=4, dims=4, base=100.0,
              scale=None, softcap=5.0, r_heads=2, r_dim=6, r_vdim=5, tau=4.0,
              rank=3, left_scale=0.7, right_scale=1.2, mlp=10):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv,
                rot=dict(base=base, dims=dims),
                scale=scale if scale is not None else dim ** -0.5,
                softcap=softcap)
    right = dict(heads=r_heads, dim=r_dim, vdim=r_vdim, tau=tau, rank=rank)
    return {"type": "parallel",
            "mixer": dict(left=left, right=right, left_scale=left_scale,
                          right_scale=right_scale),
            "mlp": None if mlp is None else dict(kind="dense", ff=mlp)}


def make_config(width=24, vocab=50, streams=2, eps=1e-5, layers=None,
                loop=None, logit_softcap=8.0):
    cfg = dict(architecture="Dunusun", vocab=vocab, width=width,
               norm=dict(eps=eps), layers=layers or [ssm_layer(), par_layer()],
               logit_softcap=logit_softcap)
    if streams is not None:
        cfg["streams"] = streams
    if loop is not None:
        cfg["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return cfg


def make_weights(cfg, seed=0, gain=1.0):
    """Random bf16-representable weights (fp32 tensors) for a config. The
    low-rank size of the decay projection is the mixer's `rank` entry (a
    size that only the tensor shapes carry; it is removed from what is
    written as config.json)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rnd(*shape, std=None):
        std = std if std is not None else gain / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def near_one(n, spread=0.2):
        return (1.0 + spread * torch.randn(n, generator=g)).bfloat16().float()

    out = {"embed": rnd(cfg["vocab"], W, std=1.0),
           "final.norm": near_one(W), "final.norm.b": rnd(W, std=0.1),
           "head": rnd(cfg["vocab"], W)}
    S = cfg.get("streams")
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        subs = [1] + ([2] if lc.get("mlp") is not None else [])
        for qn in subs:
            out[f"{p}norm{qn}"] = near_one(W)
            out[f"{p}norm{qn}.b"] = rnd(W, std=0.1)
            if S is not None:
                out[f"{p}hc{qn}.in"] = rnd(S, std=0.6) + 1.0 / S
                out[f"{p}hc{qn}.out"] = near_one(S, 0.4)
                out[f"{p}hc{qn}.mix"] = (torch.eye(S) * 0.8 + rnd(
                    S, S, std=0.15)).bfloat16().float()
        mc = lc["mixer"]
        if lc["type"] == "mamba2":
            H, P, N, G = mc["heads"], mc["vdim"], mc["state"], mc["groups"]
            inner, ch = H * P, H * P + 2 * G * N
            out[p + "mix.in"] = rnd(2 * inner + 2 * G * N + H, W)
            out[p + "mix.conv"] = rnd(ch, mc["conv"], std=0.6)
            out[p + "mix.conv.b"] = rnd(ch, std=0.2)
            out[p + "mix.dt_bias"] = rnd(H, std=1.0)
            out[p + "mix.A_log"] = (rnd(H, std=0.7) - 1.0).bfloat16().float()
            out[p + "mix.D"] = near_one(H, 0.5)
            out[p + "mix.norm"] = near_one(inner)
            out[p + "mix.o"] = rnd(W, inner)
        else:
            L, R = mc["left"], mc["right"]
            H, G, D, Dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
            lp = p + "mix.left."
            out[lp + "q"], out[lp + "k"] = rnd(H * D, W), rnd(G * D, W)
            out[lp + "v"] = rnd(G * Dv, W)
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                out[f"{lp}{n}.conv"] = rnd(rows, L["conv"], std=0.6)
            out[lp + "g"], out[lp + "o"] = rnd(H * Dv, W), rnd(W, H * Dv)
            rp = p + "mix.right."
            h2, d2, v2 = R["heads"], R["dim"], R["vdim"]
            out[rp + "q"], out[rp + "k"] = rnd(h2 * d2, W), rnd(h2 * d2, W)
            out[rp + "v"], out[rp + "g"] = rnd(h2 * v2, W), rnd(h2 * v2, W)
            out[rp + "o"] = rnd(W, h2 * v2)
            out[rp + "norm"] = near_one(v2)
            out[rp + "a1"] = rnd(R["rank"], W)
            out[rp + "a2"] = rnd(h2 * d2, R["rank"], std=1.0)
            out[rp + "a2.b"] = (rnd(h2 * d2, std=1.0) + 2.0).bfloat16().float()
        if lc.get("mlp") is not None:
            out[p + "mlp.up"] = rnd(lc["mlp"]["ff"], W)
            out[p + "mlp.down"] = rnd(W, lc["mlp"]["ff"])
    # what the file holds is what the oracle sees
    return {k: v.bfloat16().float() for k, v in out.items()}


def file_config(cfg):
    """The config as written to disk: sizes that only the tensor shapes
    carry are dropped."""
    d = json.loads(json.dumps(cfg))
    for lc in d["layers"]:
        if lc["type"] == "parallel":
            lc["mixer"]["right"].pop("rank", None)
    return d


def write_safetensors(path, tensors):
    header, blobs, off = {}, [], 0
    for name, t in tensors.items():
        raw = t.to(torch.bfloat16).contiguous().view(torch.int16).numpy() \
            .tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape),
                        "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
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
        json.dump(file_config(cfg), f)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return folder


def as_f64(weights):
    return {k: v.to(F64) for k, v in weights.items()}


def rel_err(got, want):
    """Per row: rms of the mean-free difference over the rms of `want`."""
    got, want = got.to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return torch.sqrt((d ** 2).mean(-1)) / torch.sqrt((ref ** 2).mean())
