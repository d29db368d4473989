"""Each hybrid-mixer op alone against the plain oracle (tests/hybrid_oracle.py):
CPU path always, the HIP kernels under the gpu marker. Inputs are shaped so
that a wrong key, a lost state, an edge that is one token off or a group
that is mis-scored changes the answer visibly."""
import math

import pytest
import torch

from hybrid_oracle import (F64, o_freqs, o_gnorm, o_rotate, o_route)
from xllm_service_amd.models.mixers import scaled_rope_frequencies
from xllm_service_amd.ops import hybrid as H

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, pytest.param(torch.bfloat16, marks=pytest.mark.gpu)]


def _tol(dt):
    return 3e-5 if dt == torch.float32 else 2e-2


def _close(got, want, tol):
    got, want = got.double().cpu(), want.double()
    err = float((got - want).abs().max())
    assert err <= tol * max(float(want.abs().max()), 1e-9), err


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("groups,width", [(1, 40), (4, 40), (5, 35), (2, 256)])
def test_group_rmsnorm(dev, groups, width):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(9, width, generator=g)
    x[:, :width // groups] *= 30.0          # one loud group must not leak
    w = torch.rand(width, generator=g) + 0.5
    got = H.group_rmsnorm(x.to(dev), w.to(dev), 1e-5, groups, torch.float32)
    _close(got, o_gnorm(x.to(F64), w.to(F64), 1e-5, groups), 3e-6)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("bias", [True, False])
def test_gated_norm_residual(dev, bias):
    g = torch.Generator().manual_seed(2)
    T, W, G = 7, 36, 3
    res, y, gate = (torch.randn(T, W, generator=g) for _ in range(3))
    b = torch.randn(W, generator=g) if bias else None
    w, ls = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g)
    wide = torch.randn(T, 2 * W + 5, generator=g)
    wide[:, 3:3 + W] = gate                 # gate is a strided slice
    r = res.clone().to(dev)
    H.gated_norm_residual(r, y.to(dev), wide.to(dev)[:, 3:3 + W],
                          b.to(dev) if bias else None, w.to(dev), ls.to(dev),
                          0.37, 1e-5, G)
    z = y.to(F64) * torch.sigmoid(gate.to(F64) + (b.to(F64) if bias else 0))
    want = res.to(F64) + 0.37 * ls.to(F64) * o_gnorm(z, w.to(F64), 1e-5, G)
    _close(r, want, 3e-6)


@pytest.mark.parametrize("rot", [
    dict(base=10000.0, dims=8),
    dict(base=500.0, dims=12, scaling=dict(factor=4.0, original=32, fast=16.0,
                                           slow=1.0)),
    dict(base=1e6, dims=6, scaling=dict(factor=2.5, original=4096, fast=2.0,
                                        slow=0.5)),
])
def test_scaled_frequencies(rot):
    f, mult = scaled_rope_frequencies(rot)
    fo, mo = o_freqs(rot)
    assert abs(mult - mo) < 1e-12
    _close(f, torch.tensor(fo, dtype=F64), 1e-12)
    if "scaling" in rot:                    # the ramp really blends something
        plain = [rot["base"] ** (-2.0 * i / rot["dims"])
                 for i in range(rot["dims"] // 2)]
        assert any(abs(a - b) > 1e-9 for a, b in zip(fo, plain))


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("dt", DTYPES)
def test_rotation_in_place_on_a_slice(dev, dt):
    if dev == "cpu" and dt != torch.float32:
        pytest.skip("cpu path is fp32")
    rot = dict(base=100.0, dims=6, scaling=dict(factor=2.0, original=16,
                                                fast=4.0, slow=1.0))
    f, mult = scaled_rope_frequencies(rot)
    T, Hh, D, off = 5, 3, 14, 4             # rotate dims 4..9, keep the rest
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, Hh * D + 3, generator=g).to(dt)
    pos = torch.tensor([0, 1, 7, 300, 4095])
    xd = x.clone().to(dev)
    H.rope_interleaved_(xd[:, :Hh * D].unflatten(-1, (Hh, D)), pos.to(dev),
                        f.to(dev), mult, off, rot["dims"])
    want = x.to(F64).clone()
    for t in range(T):
        for h in range(Hh):
            a = h * D + off
            want[t, a:a + 8] = o_rotate(x[t, a:a + 8].to(F64), int(pos[t]),
                                        rot)
    _close(xd, want, _tol(dt))
    assert torch.equal(xd[:, Hh * D:].cpu(), x[:, Hh * D:])


def _scrambled_tables(n_seqs, blocks_each, total, seed):
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(total, generator=g)
    t = perm[:n_seqs * blocks_each].reshape(n_seqs, blocks_each)
    return t.to(torch.int32)


def _plain_latent_attn(q, rows, scale, r, n_keys):
    s = (rows[:n_keys].to(F64) @ q.to(F64)) * scale
    return torch.softmax(s, 0) @ rows[:n_keys, :r].to(F64)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("dt", DTYPES)
def test_latent_attn_standout_keys(dev, dt):
    """One key among hundreds is made to dominate; the answer must be that
    key's latent when it is visible and must ignore it when it lies one
    position past the query — at page borders (15/16/17), tile borders
    (63/64/65), the first key and the last."""
    if dev == "cpu" and dt != torch.float32:
        pytest.skip("cpu path is fp32")
    r, rd, bs, L, Hh = 24, 8, 16, 210, 3
    W = r + rd
    g = torch.Generator().manual_seed(4)
    nblk = (L + bs - 1) // bs
    tables = _scrambled_tables(1, nblk, nblk + 5, 5)
    rows = (torch.randn(L, W, generator=g) * 0.3).to(dt)
    cache = torch.randn(nblk + 5, bs, W, generator=g).to(dt)  # stale junk
    for p in range(L):
        cache[int(tables[0, p // bs]), p % bs] = rows[p]
    cache_d = cache.to(dev)
    for star in (0, 15, 16, 17, 63, 64, 65, 128, L - 1):
        q = torch.randn(Hh, W, generator=g).to(dt) * 0.1
        q[1] = rows[star].float() * 40.0 / rows[star].float().norm() ** 2 * 3
        # decode form: the query sits at position L-1 (sees everything)
        out = torch.empty(1, Hh, r, dtype=torch.float32, device=dev)
        H.latent_attn(q[None].to(dev), cache_d, tables.to(dev), None,
                      torch.tensor([L], dtype=torch.int32, device=dev), 1.0,
                      r, out)
        for h in range(Hh):
            _close(out[0, h], _plain_latent_attn(q[h], rows, 1.0, r, L),
                   _tol(dt))
        _close(out[0, 1], rows[star, :r], 0.05)      # it is the standout key
        # prefill form: queries at star-1, star, star+1 of a 3-token chunk
        lo = max(star - 1, 0)
        hi = min(star + 2, L)
        n = hi - lo
        qq = q[None].repeat(n, 1, 1).contiguous()
        outp = torch.empty(n, Hh, r, dtype=torch.float32, device=dev)
        H.latent_attn(qq.to(dev), cache_d, tables.to(dev),
                      torch.tensor([0, n], dtype=torch.int32, device=dev),
                      torch.tensor([hi], dtype=torch.int32, device=dev), 1.0,
                      r, outp)
        for i in range(n):
            want = _plain_latent_attn(q[1], rows, 1.0, r, lo + i + 1)
            _close(outp[i, 1], want, _tol(dt))
            seen = lo + i >= star
            near = float((outp[i, 1].cpu() - rows[star, :r].float()).norm())
            assert (near < 0.3) == seen, (star, lo + i, near)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("heads,r,rd", [(1, 5, 2), (5, 70, 6), (4, 130, 0),
                                        (5, 80, 16), (3, 200, 24),
                                        (17, 512, 64), (40, 48, 8)])
def test_latent_attn_batch_of_unequal_sequences(dev, dt, heads, r, rd):
    if dev == "cpu" and dt != torch.float32:
        pytest.skip("cpu path is fp32")
    bs, W = 16, r + rd
    g = torch.Generator().manual_seed(6)
    lens, chunk = [70, 3, 33, 16], [5, 3, 2, 16]
    nb = 6
    tables = _scrambled_tables(len(lens), nb, len(lens) * nb + 2, 7)
    cache = torch.randn(len(lens) * nb + 2, bs, W, generator=g).to(dt)
    q = torch.randn(sum(chunk), heads, W, generator=g).to(dt)
    cu = torch.tensor([0] + list(torch.tensor(chunk).cumsum(0)),
                      dtype=torch.int32)
    out = torch.empty(sum(chunk), heads, r, dtype=torch.float32, device=dev)
    H.latent_attn(q.to(dev), cache.to(dev), tables.to(dev), cu.to(dev),
                  torch.tensor(lens, dtype=torch.int32, device=dev), 0.3, r,
                  out)
    for s, (L, c) in enumerate(zip(lens, chunk)):
        rows = torch.stack([cache[int(tables[s, p // bs]), p % bs]
                            for p in range(L)])
        for i in range(c):
            for h in range(heads):
                want = _plain_latent_attn(q[int(cu[s]) + i, h], rows, 0.3, r,
                                          L - c + i + 1)
                _close(out[int(cu[s]) + i, h], want, _tol(dt))


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("dt", DTYPES)
def test_latent_kv_store(dev, dt):
    if dev == "cpu" and dt != torch.float32:
        pytest.skip("cpu path is fp32")
    rot = dict(base=50.0, dims=4, scaling=dict(factor=2.0, original=8,
                                               fast=2.0, slow=1.0))
    f, mult = scaled_rope_frequencies(rot)
    r, rd, bs = 10, 6, 16                   # rot dims 4 of a 6-wide tail
    g = torch.Generator().manual_seed(8)
    T = 6
    dkv = torch.randn(T, r + rd + 2, generator=g).to(dt)
    w = torch.rand(r, generator=g) + 0.5
    pos = torch.tensor([0, 1, 15, 16, 17, 900])
    slots = torch.tensor([5, 4, -1, 47, 16, 15])
    cache = torch.full((3, bs, r + rd), 7.0, dtype=dt)
    cd = cache.clone().to(dev)
    H.latent_kv_store(dkv.to(dev)[:, :r + rd], w.to(dev), 1e-5, pos.to(dev),
                      f.to(dev), mult, rot["dims"], cd, slots.to(dev), r)
    flat = cd.view(-1, r + rd).cpu()
    for t in range(T):
        if slots[t] < 0:
            continue
        x = dkv[t].to(F64)
        want = torch.cat([o_gnorm(x[:r], w.to(F64), 1e-5, 1),
                          o_rotate(x[r:r + rd], int(pos[t]), rot)])
        _close(flat[int(slots[t])], want, _tol(dt))
    untouched = [i for i in range(3 * bs) if i not in slots.tolist()]
    assert torch.all(flat[untouched] == 7.0)


def _plain_decay(q, k, v, a, S):
    silu = lambda z: z * torch.sigmoid(z)
    q, k, v = silu(q.to(F64)), silu(k.to(F64)), silu(v.to(F64))
    out = []
    for t in range(q.shape[0]):
        S = a * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out), S


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("heads,d,vd", [(2, 8, 8), (3, 20, 17), (1, 64, 40)])
def test_decay_attn_state_through_portions(dev, heads, d, vd):
    """One sequence cut at 1/15/16/17-token edges, a stale slot that must be
    ignored at ctx 0, a slotless row, and decode rows — all against the
    token recurrence."""
    g = torch.Generator().manual_seed(9)
    T = 60
    wide = torch.randn(T, heads * (2 * d + vd) + 3, generator=g)
    q, k = wide[:, :heads * d], wide[:, heads * d:2 * heads * d]
    v = wide[:, 2 * heads * d:2 * heads * d + vd * heads]
    a = torch.tensor([0.999, 0.6, 0.9][:heads])
    state = torch.randn(3, heads, d, vd, generator=g).to(dev)   # stale
    junk = state.clone()
    wd, ad = wide.to(dev), a.to(dev)
    qd, kd = wd[:, :heads * d], wd[:, heads * d:2 * heads * d]
    vdv = wd[:, 2 * heads * d:2 * heads * d + vd * heads]
    got = torch.empty(T, heads, vd, dtype=torch.float32, device=dev)
    at = 0
    for n in (1, 15, 16, 17, 2, 1, 1, 7):
        sl = slice(at, at + n)
        i32 = dict(dtype=torch.int32, device=dev)
        cu = None if (n == 1 and at > 0) else torch.tensor([0, n], **i32)
        H.decay_attn(qd[sl], kd[sl], vdv[sl], ad, state,
                     torch.tensor([1], **i32), cu, torch.tensor([at], **i32),
                     got[sl])
        at += n
    assert at == T
    for h in range(heads):
        want, S = _plain_decay(q[:, h * d:(h + 1) * d], k[:, h * d:(h + 1) * d],
                               v[:, h * vd:(h + 1) * vd], float(a[h]),
                               torch.zeros(d, vd, dtype=F64))
        _close(got[:, h], want, 2e-5)
        _close(state[1, h], S, 2e-5)
    assert torch.equal(state[0], junk[0]) and torch.equal(state[2], junk[2])
    # two rows in one call: slot -1 runs from zero and stores nothing
    i32 = dict(dtype=torch.int32, device=dev)
    o2 = torch.empty(2, heads, vd, dtype=torch.float32, device=dev)
    before = state.clone()
    H.decay_attn(qd[:2], kd[:2], vdv[:2], ad, state, torch.tensor([-1, 2], **i32),
                 None, torch.tensor([9, 0], **i32), o2)
    for h in range(heads):
        for row in range(2):
            want, S = _plain_decay(q[row:row + 1, h * d:(h + 1) * d],
                                   k[row:row + 1, h * d:(h + 1) * d],
                                   v[row:row + 1, h * vd:(h + 1) * vd],
                                   float(a[h]), torch.zeros(d, vd, dtype=F64))
            _close(o2[row, h], want[0], 2e-5)
        _close(state[2, h], S, 2e-5)
    assert torch.equal(state[:2], before[:2])


@pytest.mark.parametrize("dev", DEVS)
def test_router_group_limit_beats_single_best(dev):
    """The expert with the highest score sits in a group whose two best sum
    lower than another group's: it must not be chosen."""
    E, W = 6, 6
    wr = torch.eye(E, W) * 1.0
    h = torch.tensor([[4.0, -6.0, -6.0, 2.0, 1.5, -6.0],      # groups of 3
                      [-6.0, 1.0, 0.9, 3.0, -6.0, -6.0]])
    ids, wts = H.moe_route(h.to(dev), wr.to(dev), 2, 2, 1)
    s = torch.sigmoid(h.to(F64))
    assert sorted(ids[0].tolist()) == [3, 4]
    assert sorted(ids[1].tolist()) == [1, 2]
    for t in range(2):
        for j in range(2):
            assert abs(float(wts[t, j]) - float(s[t, int(ids[t, j])])) < 1e-6
    # without groups the plain top-2 wins
    ids, _ = H.moe_route(h.to(dev), wr.to(dev), 2, 1, 1)
    assert sorted(ids[0].tolist()) == [0, 3]
    assert sorted(ids[1].tolist()) == [1, 3]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("E,top,count,keep", [(12, 3, 4, 2), (8, 1, 8, 3),
                                              (9, 4, 1, 1), (66, 6, 11, 4)])
def test_router_random(dev, E, top, count, keep):
    g = torch.Generator().manual_seed(10)
    W, T = 40, 23
    h = torch.randn(T, W, generator=g)
    wr = torch.randn(E, W, generator=g) * 0.3
    ids, wts = H.moe_route(h.to(dev), wr.to(dev), top, count, keep)
    rc = dict(experts=E, top=top, groups=dict(count=count, keep=keep))
    for t in range(T):
        s = torch.sigmoid(wr.to(F64) @ h[t].to(F64))
        assert sorted(ids[t].tolist()) == sorted(o_route(s.tolist(), rc))
        for j in range(top):
            assert abs(float(wts[t, j]) - float(s[int(ids[t, j])])) < 1e-6


@pytest.mark.parametrize("dev", DEVS)
def test_combine_and_silu_mul(dev):
    g = torch.Generator().manual_seed(11)
    y = torch.randn(31, 20, generator=g)
    rows = torch.randint(0, 31, (9, 3), generator=g).to(torch.int32)
    wts = torch.rand(9, 3, generator=g)
    got = H.moe_combine(y.to(dev), rows.to(dev), wts.to(dev), 9)
    want = (y.to(F64)[rows.long()] * wts.to(F64)[:, :, None]).sum(1)
    _close(got, want, 3e-6)
    x = torch.randn(2, 5, 14, generator=g)
    z = x.to(F64)
    _close(H.silu_mul(x.to(dev)), z[..., :7] * torch.sigmoid(z[..., :7])
           * z[..., 7:], 3e-6)


@pytest.mark.parametrize("dev", DEVS)
def test_norm_sigmoid_gate(dev):
    g = torch.Generator().manual_seed(12)
    o, gate = torch.randn(6, 30, generator=g), torch.randn(6, 30, generator=g)
    w = torch.rand(30, generator=g) + 0.5
    got = H.norm_sigmoid_gate(o.to(dev), w.to(dev), gate.to(dev), 1e-5,
                              torch.float32)
    want = o_gnorm(o.to(F64), w.to(F64), 1e-5, 1) * torch.sigmoid(gate.to(F64))
    _close(got, want, 3e-6)
    got = H.norm_sigmoid_gate(o.to(dev), None, gate.to(dev), 1e-5,
                              torch.float32)
    _close(got, o.to(F64) * torch.sigmoid(gate.to(F64)), 3e-6)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("heads,r,rd", [(2, 40, 8), (19, 128, 32),
                                        (24, 512, 64), (40, 48, 8),
                                        (70, 32, 0)])
def test_latent_attn_decode_rows_of_unequal_context(dev, dt, heads, r, rd):
    """Decode rows whose contexts differ widely (the kernel may split long
    contexts over several workgroups and merge the parts)."""
    if dev == "cpu" and dt != torch.float32:
        pytest.skip("cpu path is fp32")
    bs, W = 16, r + rd
    g = torch.Generator().manual_seed(13)
    lens = [1, 700, 33, 64, 65, 257]
    nb = (max(lens) + bs - 1) // bs
    tables = _scrambled_tables(len(lens), nb, len(lens) * nb + 3, 14)
    cache = (torch.randn(len(lens) * nb + 3, bs, W, generator=g) * 0.5).to(dt)
    q = torch.randn(len(lens), heads, W, generator=g).to(dt)
    out = torch.empty(len(lens), heads, r, dtype=torch.float32, device=dev)
    H.latent_attn(q.to(dev), cache.to(dev), tables.to(dev), None,
                  torch.tensor(lens, dtype=torch.int32, device=dev), 0.2, r,
                  out)
    for s, L in enumerate(lens):
        rows = torch.stack([cache[int(tables[s, p // bs]), p % bs]
                            for p in range(L)])
        for h in range(heads):
            _close(out[s, h], _plain_latent_attn(q[s, h], rows, 0.2, r, L),
                   _tol(dt))


@pytest.mark.parametrize("dev", DEVS)
def test_decay_attn_long_portions(dev):
    """Portions long enough for the chunk-parallel path on the GPU: two
    sequences in one call, one continuing from a stored state, lengths that
    end inside a chunk; then a second portion continues both."""
    heads, d, vd = 2, 16, 24
    g = torch.Generator().manual_seed(15)
    lens1, lens2 = [700, 301], [129, 260]
    T1, T2 = sum(lens1), sum(lens2)
    wide = torch.randn(T1 + T2, heads * (2 * d + vd), generator=g) * 0.7
    a = torch.tensor([0.99, 0.8])
    state = torch.zeros(3, heads, d, vd)
    state[2] = torch.randn(heads, d, vd, generator=g)
    init = state.clone()
    sd, wd, ad = state.to(dev), wide.to(dev), a.to(dev)
    i32 = dict(dtype=torch.int32, device=dev)
    o1 = torch.empty(T1, heads, vd, dtype=torch.float32, device=dev)
    x = wd[:T1]
    H.decay_attn(x[:, :heads * d], x[:, heads * d:2 * heads * d],
                 x[:, 2 * heads * d:], ad, sd, torch.tensor([0, 2], **i32),
                 torch.tensor([0, 700, 1001], **i32),
                 torch.tensor([0, 5], **i32), o1, max_q_len=700)
    o2 = torch.empty(T2, heads, vd, dtype=torch.float32, device=dev)
    x = wd[T1:]
    H.decay_attn(x[:, :heads * d], x[:, heads * d:2 * heads * d],
                 x[:, 2 * heads * d:], ad, sd, torch.tensor([0, 2], **i32),
                 torch.tensor([0, 129, 389], **i32),
                 torch.tensor([700, 306], **i32), o2, max_q_len=260)
    seqs = [(torch.cat([wide[:700], wide[T1:T1 + 129]]), 0, False),
            (torch.cat([wide[700:T1], wide[T1 + 129:]]), 2, True)]
    got = [torch.cat([o1[:700], o2[:129]]), torch.cat([o1[700:], o2[129:]])]
    for (x, slot, carried), o in zip(seqs, got):
        for h in range(heads):
            S0 = init[slot, h].to(F64) if carried else torch.zeros(d, vd,
                                                                   dtype=F64)
            want, S = _plain_decay(
                x[:, h * d:(h + 1) * d],
                x[:, heads * d + h * d:heads * d + (h + 1) * d],
                x[:, 2 * heads * d + h * vd:2 * heads * d + (h + 1) * vd],
                float(a[h]), S0)
            _close(o[:, h], want, 5e-5)
            _close(sd[slot, h], S, 5e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("skew", [False, True])
def test_routed_experts_three_execution_shapes_agree(dev, skew):
    """All-experts batched, padded-by-expert and expert-by-expert execution
    give the same mixture; `skew` sends most tokens to one expert so the
    padded shape is refused."""
    from xllm_service_amd.models.moe import RoutedExperts
    from hybrid_oracle import o_experts
    g = torch.Generator().manual_seed(16)
    W, ff, E, top, T = 24, 10, 8, 2, 150
    m = RoutedExperts(W, ff, E, top, 4, 2, torch.float32)
    with torch.no_grad():
        m.router.copy_(torch.randn(E, W, generator=g) * 0.5)
        if skew:
            m.router[0] += 3.0 * torch.ones(W) / math.sqrt(W)
        m.w_gate_up.copy_(torch.randn(E, 2 * ff, W, generator=g) * 0.3)
        m.w_down.copy_(torch.randn(E, W, ff, generator=g) * 0.3)
    h = torch.randn(T, W, generator=g) + (2.0 / math.sqrt(W) if skew else 0.0)
    wt = {"router": m.router.detach().to(F64)}
    for e in range(E):
        wt[f"e{e}.gate"] = m.w_gate_up[e, :ff].detach().to(F64)
        wt[f"e{e}.up"] = m.w_gate_up[e, ff:].detach().to(F64)
        wt[f"e{e}.down"] = m.w_down[e].detach().to(F64)
    fc = dict(router=dict(experts=E, top=top, groups=dict(count=4, keep=2)))
    want = o_experts(wt, "", fc, h.to(F64))
    m = m.to(dev)
    with torch.no_grad():
        sorted_out = m(h.to(dev))
        m.dense_max_tokens = 10 ** 6
        dense_out = m(h.to(dev))
    _close(sorted_out, want, 2e-5)
    _close(dense_out, want, 2e-5)
