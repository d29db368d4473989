"""The mechanisms of the Dunusun decoder one at a time: the op layer
(xllm_service_amd.ops.hybrid; fp32 torch on the CPU, HIP kernels under the gpu
marker, fp32 and bf16 storage) against plain fp64 loops written here and the
functions of tests/dunusun_oracle.py. Inputs are made so that a fault shows:
a far key whose score stands out, scores large enough for the cap to bite,
portions shorter than a filter, slots that still hold another sequence."""
import math

import pytest
import torch

from dunusun_oracle import F64, o_conv, o_layernorm, o_rotate, o_silu
from xllm_service_amd.ops import hybrid as hops

TARGETS = [("cpu", torch.float32),
           pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
           pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]


def _tol(target):
    return 2e-5 if target[1] == torch.float32 else 2e-2


def _close(got, want, target, what="", scale=1.0):
    got, want = got.detach().cpu().to(F64), want.to(F64)
    err = float((got - want).abs().max() / max(float(want.abs().max()), 1e-9))
    assert err < _tol(target) * scale, (what, err)


def _rnd(g, *shape, dtype=torch.float32, std=1.0):
    """Random values that bf16 holds exactly (so both storage types see the
    same inputs as the fp64 loops)."""
    return (torch.randn(*shape, generator=g) * std).bfloat16().to(dtype)


def _i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


# ------------------------------------------------------------ residual streams
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("S,W", [(1, 20), (3, 70), (8, 257), (2, 1288)])
def test_streams_read_and_write(target, S, W):
    dev, dt = target
    g = torch.Generator().manual_seed(S * 100 + W)
    T = 5
    x = torch.randn(T, S, W, generator=g) * 3 + 1.0
    w_in, w_out = torch.randn(S, generator=g), torch.randn(S, generator=g)
    mix = torch.randn(S, S, generator=g)
    nw, nb = torch.randn(W, generator=g), torch.randn(W, generator=g)
    y1, y2 = _rnd(g, T, W, dtype=dt), _rnd(g, T, W, dtype=dt)
    xd = x.clone().to(dev)
    h = hops.streams_mix_norm(xd, w_in.to(dev), nw.to(dev), nb.to(dev), 1e-5,
                              dt)
    u = torch.einsum("tsw,s->tw", x.to(F64), w_in.to(F64))
    _close(h, o_layernorm(u, nw.to(F64), nb.to(F64), 1e-5), target, "read")
    # plain sum when no read weights are given
    h = hops.streams_mix_norm(xd, None, nw.to(dev), nb.to(dev), 1e-5, dt)
    _close(h, o_layernorm(x.to(F64).sum(1), nw.to(F64), nb.to(F64), 1e-5),
           target, "sum")
    hops.streams_update_(xd, mix.to(dev), w_out.to(dev), y1.to(dev), 0.7,
                         y2.to(dev), -1.3)
    y = 0.7 * y1.to(F64) + -1.3 * y2.to(F64)
    want = torch.stack([
        sum(mix[s, j].to(F64) * x[:, s].to(F64) for s in range(S))
        + w_out[j].to(F64) * y for j in range(S)], 1)
    _close(xd, want, ("", torch.float32), "write")
    # the write fused with the next sublayer's read
    xf = x.clone().to(dev)
    w2 = torch.randn(S, generator=g)
    h = hops.streams_update_mix_norm_(xf, mix.to(dev), w_out.to(dev),
                                      y1.to(dev), 0.7, y2.to(dev), -1.3,
                                      w2.to(dev), nw.to(dev), nb.to(dev), 1e-5)
    _close(xf, want, ("", torch.float32), "fused write")
    u = torch.einsum("tsw,s->tw", want, w2.to(F64))
    _close(h, o_layernorm(u, nw.to(F64), nb.to(F64), 1e-5), target, "fused")
    # identity mixing = the plain residual sum
    x1 = x[:, :1].clone().to(dev)
    hops.streams_update_(x1, None, None, y1.to(dev))
    _close(x1[:, 0], x[:, 0].to(F64) + y1.to(F64), ("", torch.float32), "res")


@pytest.mark.parametrize("target", TARGETS)
def test_relu_sq_and_softcap(target):
    dev, dt = target
    g = torch.Generator().manual_seed(3)
    x = _rnd(g, 7, 33, dtype=dt, std=4.0)
    want = torch.relu(x.to(F64)) ** 2
    _close(hops.relu_sq_(x.clone().to(dev)), want, target)
    big = _rnd(g, 4, 50, dtype=dt, std=40.0)     # far into the flat part
    got = hops.softcap(big.to(dev), 30.0)
    assert got.dtype == torch.float32
    _close(got, 30.0 * torch.tanh(big.to(F64) / 30.0), ("", torch.float32))
    assert float(got.abs().max()) <= 30.0


# ------------------------------------------------------------ gated group norm
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("groups,shared,silu,first", [
    (1, False, True, True), (4, False, True, True), (3, True, True, False),
    (1, False, False, False), (6, True, False, True)])
def test_gated_group_norm(target, groups, shared, silu, first):
    dev, dt = target
    g = torch.Generator().manual_seed(groups)
    rows, gs = 6, 10
    n = groups * gs
    o = torch.randn(rows, n, generator=g) * 2
    gate = _rnd(g, rows, n + 3, dtype=dt)[:, 3:]            # a row view
    w = torch.randn(gs if shared else n, generator=g)
    got = hops.gated_group_norm(o.to(dev), w.to(dev), gate.to(dev), 1e-5,
                                groups, act_silu=silu, gate_first=first,
                                out_dtype=dt)
    a = o_silu(gate.to(F64)) if silu else torch.sigmoid(gate.to(F64))
    z = o.to(F64) * a if first else o.to(F64)
    zz = z.view(rows, groups, gs)
    zz = zz / torch.sqrt((zz ** 2).mean(-1, keepdim=True) + 1e-5)
    wf = w.to(F64).repeat(groups) if shared else w.to(F64)
    z = zz.reshape(rows, n) * wf
    if not first:
        z = z * a
    _close(got, z, target)


# ------------------------------------------------------------ short convolution
def _conv_case(target, C, taps, portions, heads=1, rot_dims=0, bias=True,
               silu=False, seed=0, paged=False):
    """Two sequences through portions with carried state; sequence B starts
    on the slot sequence A used. portions: list of (lenA, lenB) per step,
    0 = absent."""
    dev, dt = target
    g = torch.Generator().manual_seed(seed)
    hd = C // heads
    LA = sum(a for a, _ in portions)
    LB = sum(b for _, b in portions)
    xs = {"A": _rnd(g, LA, C + 2, dtype=dt)[:, 1:C + 1],   # row views
          "B": _rnd(g, LB, C + 2, dtype=dt)[:, 1:C + 1]}
    w = _rnd(g, C, taps, dtype=dt, std=0.7)
    b = _rnd(g, C, dtype=dt) if bias else None
    rot = dict(base=50.0, dims=rot_dims)
    inv = torch.tensor([50.0 ** (-2.0 * i / max(rot_dims, 1))
                        for i in range(rot_dims // 2)], dtype=F64)
    want = {}
    for k, x in xs.items():
        y = o_conv(x.to(F64), w.to(F64), None if b is None else b.to(F64))
        if silu:
            y = o_silu(y)
        if rot_dims:
            y = y.view(-1, heads, hd).clone()
            for t in range(y.shape[0]):
                for h in range(heads):
                    y[t, h] = o_rotate(y[t, h], t, rot)
            y = y.reshape(-1, C)
        want[k] = y
    state = torch.full((2, taps - 1, C + 3), 7.0, dtype=dt, device=dev)
    bs, nblk = 4, (max(LA, LB) + 3) // 4
    cache = torch.zeros(2 * nblk, heads, bs, hd, dtype=dt, device=dev)
    got = {"A": [], "B": []}
    at = {"A": 0, "B": 0}
    slot_of = {"A": 1, "B": 1 if LA == 0 else 0}
    for la, lb in portions:
        rows, cu, ctx, slots, names = [], [0], [], [], []
        for k, n in (("A", la), ("B", lb)):
            if n:
                rows.append(xs[k][at[k]:at[k] + n])
                cu.append(cu[-1] + n)
                ctx.append(at[k])
                slots.append(slot_of[k])
                names.append((k, n))
        x = torch.cat(rows).to(dev)
        x = torch.cat([x.new_zeros(x.shape[0], 2), x], 1)[:, 2:]   # strided
        pos = torch.cat([torch.arange(at[k], at[k] + n) for k, n in names])
        sm = torch.cat([(0 if k == "A" else nblk) * bs
                        + torch.arange(at[k], at[k] + n) for k, n in names])
        decode = all(n == 1 for _, n in names)
        kw = dict(act_silu=silu, rot_dims=rot_dims, positions=pos.to(dev),
                  inv_freq=inv.to(dev) if rot_dims else None)
        if paged:
            kw.update(cache=cache, slot_mapping=sm.to(dev))
        y = hops.short_conv(x, w.to(dev), None if b is None else b.to(dev),
                            state, 2, _i32(slots, dev),
                            None if decode else _i32(cu, dev), _i32(ctx, dev),
                            heads, hd, **kw)
        # the state moves once every reader of the old one has run
        full = torch.cat([x.new_zeros(x.shape[0], 2), x,
                          x.new_zeros(x.shape[0], 1)], 1)
        hops.short_conv_state_(state, full, _i32(slots, dev),
                               None if decode else _i32(cu, dev))
        o = 0
        for k, n in names:
            if not paged:
                got[k].append(y[o:o + n])
            o += n
            at[k] += n
    for k in ("A", "B"):
        L = want[k].shape[0]
        if not L:
            continue
        if paged:
            off = 0 if k == "A" else nblk
            blk = cache[off:off + nblk].permute(0, 2, 1, 3).reshape(-1, C)
            _close(blk[:L], want[k], target, k)
        else:
            _close(torch.cat(got[k]), want[k], target, k)


@pytest.mark.parametrize("target", TARGETS)
def test_short_conv_portions_and_slots(target):
    # portions shorter than the filter, single tokens, one long portion
    _conv_case(target, 6, 4, [(1, 0), (2, 5), (1, 1), (1, 1), (7, 2), (1, 0)],
               seed=1)
    _conv_case(target, 5, 3, [(9, 1), (1, 1), (1, 3)], silu=True, seed=2)
    _conv_case(target, 7, 2, [(3, 0), (2, 2)], bias=False, seed=3)
    # a filter of one tap keeps no state
    _conv_case(target, 4, 1, [(3, 2), (1, 1)], seed=4)
    # a long filter against short sequences
    _conv_case(target, 3, 9, [(2, 1), (2, 1), (1, 1), (6, 6)], seed=5)


@pytest.mark.parametrize("target", TARGETS)
def test_short_conv_rotation_and_paged_store(target):
    # heads of odd width, part of each head turned
    _conv_case(target, 15, 4, [(6, 2), (1, 1), (5, 3)], heads=3, rot_dims=4,
               bias=False, seed=6)
    # every dimension turned; straight into a paged cache
    _conv_case(target, 16, 3, [(5, 2), (1, 1), (9, 7)], heads=2, rot_dims=8,
               bias=False, seed=7, paged=True)
    _conv_case(target, 12, 4, [(3, 3), (1, 1)], heads=2, rot_dims=0,
               bias=False, seed=8, paged=True)


# ------------------------------------------------------- gated recurrences
def _plain_recurrence(a, k, v, q, skip=None):
    """a [T, D], k, q [T, D], v [T, Dv] -> o [T, Dv] from a zero state."""
    T, D = k.shape
    S = torch.zeros(D, v.shape[1], dtype=F64)
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        S = a[t][:, None] * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
        if skip is not None:
            out[t] += skip * v[t]
    return out


def _recurrence_case(target, kind, H, G, D, Dv, lens, portions, seed=0,
                     fast_decay=False):
    """lens: length per sequence; portions: per step a list of
    (sequence, tokens). Every sequence owns a slot that held junk."""
    dev, dt = target
    g = torch.Generator().manual_seed(seed)
    n_seq = len(lens)
    q = [_rnd(g, L, G * D, dtype=dt) for L in lens]
    k = [_rnd(g, L, G * D, dtype=dt, std=0.5) for L in lens]
    v = [_rnd(g, L, H * Dv, dtype=dt) for L in lens]
    if kind == 0:
        gt = [_rnd(g, L, H, dtype=dt) for L in lens]
        p0 = torch.randn(H, generator=g)
        p1 = torch.randn(H, generator=g) * 0.5 + (1.0 if fast_decay else -1.5)
        p2 = torch.randn(H, generator=g)
        c0, c1 = 0.0, 1.0
    else:
        gt = [_rnd(g, L, H * D, dtype=dt, std=2.0) for L in lens]
        p0 = torch.randn(H * D, generator=g) + (0.0 if fast_decay else 3.0)
        p1 = p2 = None
        c0, c1 = (1.0 if fast_decay else 1.0 / 8.0), D ** -0.5
    want = []
    for s, L in enumerate(lens):
        o = torch.zeros(L, H, Dv, dtype=F64)
        for h in range(H):
            kg = h // (H // G)
            qq = q[s].to(F64)[:, kg * D:(kg + 1) * D]
            kk = k[s].to(F64)[:, kg * D:(kg + 1) * D]
            vv = v[s].to(F64)[:, h * Dv:(h + 1) * Dv]
            if kind == 0:
                x = gt[s].to(F64)[:, h] + p0[h].to(F64)
                dtv = torch.where(x > 30, x, torch.log1p(torch.exp(x)))
                a = torch.exp(-math.exp(float(p1[h])) * dtv)[:, None] \
                    .expand(L, D)
                o[:, h] = _plain_recurrence(a, kk * dtv[:, None], vv, qq,
                                            float(p2[h]))
            else:
                z = gt[s].to(F64)[:, h * D:(h + 1) * D] \
                    + p0.to(F64)[h * D:(h + 1) * D]
                a = torch.sigmoid(z) ** c0
                o[:, h] = _plain_recurrence(a, kk, vv, qq * c1)
        want.append(o)
    state = torch.full((n_seq + 1, H, D, Dv), 3.0, device=dev)
    at = [0] * n_seq
    got = [[] for _ in lens]
    for step in portions:
        cu = [0]
        for s, n in step:
            cu.append(cu[-1] + n)
        decode = all(n == 1 for _, n in step) and all(at[s] > 0
                                                      for s, _ in step)
        cat = lambda xs: torch.cat(                       # noqa: E731
            [xs[s][at[s]:at[s] + n] for s, n in step]).to(dev)
        out = torch.empty(cu[-1], H, Dv, device=dev)
        hops.gated_recurrence(
            kind, cat(q), cat(k), cat(v), cat(gt), p0.to(dev),
            None if p1 is None else p1.to(dev),
            None if p2 is None else p2.to(dev), c0, c1, state,
            _i32([s + 1 for s, _ in step], dev),
            None if decode else _i32(cu, dev),
            _i32([at[s] for s, _ in step], dev), G, out,
            max_q_len=max(n for _, n in step))
        for i, (s, n) in enumerate(step):
            got[s].append(out[cu[i]:cu[i + 1]])
            at[s] += n
    assert at == list(lens)
    for s in range(n_seq):
        _close(torch.cat(got[s]), want[s], target, (kind, s), scale=4.0)
    assert float(state[0].min()) == 3.0            # a slot nobody owns


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("kind", [0, 1])
def test_recurrence_portions_and_decoding(target, kind):
    H, G = (4, 2) if kind == 0 else (3, 3)
    # widths that fill neither a row group nor a column slice
    _recurrence_case(target, kind, H, G, 5, 7, [30, 9],
                     [[(0, 7), (1, 2)], [(0, 1), (1, 1)], [(0, 2), (1, 6)],
                      [(0, 1)], [(0, 19)]], seed=kind)
    # value width on the vector decode path; long decoding
    _recurrence_case(target, kind, H, G, 20, 8, [40],
                     [[(0, 3)]] + [[(0, 1)]] * 37, seed=10 + kind)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("fast", [False, True])
def test_recurrence_long_chunks(target, kind, fast):
    """Chunks long enough for the piece-parallel path, cut at odd places,
    beside a short sequence; slow and fast forgetting."""
    H, G = (2, 1) if kind == 0 else (2, 2)
    _recurrence_case(target, kind, H, G, 18, 16, [700, 5],
                     [[(0, 300), (1, 4)], [(0, 1), (1, 1)], [(0, 399)]],
                     seed=20 + kind, fast_decay=fast)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("cols", ["1", "4"])
def test_recurrence_wide_values(target, kind, cols, monkeypatch):
    """Wide value rows, with one and with four columns per thread (the
    kernel picks by grid size; the knob fixes it), whole chunks and pieces;
    a value width that leaves the last column group part empty."""
    monkeypatch.setenv("XLLM_RECURRENCE_COLS", cols)
    H, G = (2, 1) if kind == 0 else (2, 2)
    _recurrence_case(target, kind, H, G, 12, 72, [330, 40],
                     [[(0, 290), (1, 39)], [(0, 1), (1, 1)], [(0, 39)]],
                     seed=30 + kind)
    _recurrence_case(target, kind, H, G, 33, 50, [21],
                     [[(0, 20)], [(0, 1)]], seed=40 + kind)


# ------------------------------------------------------- soft-capped attention
def _attn_case(target, H, G, D, Dv, L, cap, scale, chunks, standout=None,
               seed=0):
    """One sequence of L tokens on scattered pages, queries run in chunks;
    standout = (query position, key position) whose score is made large."""
    dev, dt = target
    g = torch.Generator().manual_seed(seed)
    q = _rnd(g, L, H, D, dtype=dt)
    k = _rnd(g, L, G, D, dtype=dt)
    v = _rnd(g, L, G, Dv, dtype=dt)
    if standout:
        qi, kj = standout
        k[kj] = k[kj] * 4
        q[qi] = k[kj].repeat_interleave(H // G, 0) * 2
    bs = 16
    nblk = (L + bs - 1) // bs
    perm = torch.randperm(nblk + 3, generator=g)[:nblk]
    kc = torch.zeros(nblk + 3, G, bs, D, dtype=dt)
    vc = torch.zeros(nblk + 3, G, bs, Dv, dtype=dt)
    for t in range(L):
        kc[perm[t // bs], :, t % bs] = k[t]
        vc[perm[t // bs], :, t % bs] = v[t]
    want = torch.zeros(L, H, Dv, dtype=F64)
    for h in range(H):
        kg = h // (H // G)
        for t in range(L):
            sc = (k[:t + 1, kg].to(F64) @ q[t, h].to(F64)) * scale
            if cap:
                sc = cap * torch.tanh(sc / cap)
            want[t, h] = torch.softmax(sc, 0) @ v[:t + 1, kg].to(F64)
    tables = perm[None].to(torch.int32).to(dev)
    kc, vc = kc.to(dev), vc.to(dev)
    got, at = [], 0
    for n in chunks:
        out = torch.empty(n, H, Dv, device=dev)
        decode = n == 1 and at > 0
        hops.capped_attn(q[at:at + n].reshape(n, H * D).to(dev), kc, vc,
                         tables, None if decode else _i32([0, n], dev),
                         _i32([at + n], dev), H, scale, cap or 0.0, out)
        got.append(out)
        at += n
    assert at == L
    got = torch.cat(got)
    _close(got, want, target, (H, G, D, Dv, cap), scale=2.0)
    return got, want, v


@pytest.mark.parametrize("target", TARGETS)
def test_attention_sizes_and_groups(target):
    _attn_case(target, 4, 2, 8, 6, 37, 5.0, 0.4, [20, 1, 1, 15], seed=1)
    _attn_case(target, 3, 1, 5, 70, 20, None, 0.3, [1, 1, 18], seed=2)
    _attn_case(target, 2, 2, 40, 9, 33, 50.0, 0.1, [33], seed=3)
    _attn_case(target, 6, 3, 16, 16, 70, 2.0, 1.0, [64, 2, 1, 1, 1, 1], seed=4)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 128, 256), (2, 1, 128, 128),
                                      (2, 2, 256, 256), (40, 2, 64, 64),
                                      (36, 1, 32, 64),
                                      (3, 1, 24, 136)])
def test_attention_wide_heads(target, H, G, D, Dv):
    """Head widths of every size class of the matrix-core kernel, prompt
    chunks cut inside a key tile and decoding with many heads per group."""
    _attn_case(target, H, G, D, Dv, 75, 4.0, D ** -0.5, [33, 31, 9, 1, 1],
               seed=D + Dv)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("key", [0, 3, 15, 16, 17, 63, 64, 255, 256])
def test_attention_far_key_stands_out(target, key):
    """One far key carries almost all the weight of the last query, in a
    prompt chunk and in decoding; without a cap the output is that key's
    value row."""
    L = 300
    for chunks in ([L], [L - 1, 1]):
        got, want, v = _attn_case(target, 2, 1, 16, 8, L, None, 0.5, chunks,
                                  standout=(L - 1, key), seed=key)
        row = got[L - 1, 0].cpu().to(F64)
        assert float((row - v[key, 0].to(F64)).abs().max()) < 0.05


@pytest.mark.parametrize("target", TARGETS)
def test_attention_cap_limits_a_standout_score(target):
    """With the cap the standout score saturates, so the far key shares the
    weight: the result must differ clearly from the uncapped one and match
    the plain loops."""
    L = 100
    capped, _, v = _attn_case(target, 2, 1, 16, 8, L, 3.0, 0.5, [L],
                              standout=(L - 1, 7), seed=5)
    row = capped[L - 1, 0].cpu().to(F64)
    assert float((row - v[7, 0].to(F64)).abs().max()) > 0.2
