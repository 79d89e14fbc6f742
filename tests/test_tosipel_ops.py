"""The mechanisms of the Tosipel decoder one at a time: the op layer
(xllm_service_amd.ops.hybrid; fp32 torch on the CPU, HIP kernels under the gpu
marker, fp32 and bf16 storage) against the plain fp64 functions of
tests/tosipel_oracle.py. Inputs are made so that a fault shows: one key whose
score stands out just inside or just outside the window, at page and tile
borders, or far back; a sink that dominates; a state slot that still holds
another sequence."""
import math

import pytest
import torch

from tosipel_oracle import (F64, o_attend, o_delta_core, o_gelu_tanh, o_rms,
                            o_rotate_halves, o_sigmoid)
from xllm_service_amd.ops import hybrid as hops

TARGETS = [("cpu", torch.float32),
           pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
           pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]
BS = 16                                    # page size of the engine's pool


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


# ------------------------------------------------- post norm, gates, GELU
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("W", [20, 257, 1288])
def test_post_norm_residual(target, W):
    dev, dt = target
    g = torch.Generator().manual_seed(W)
    T = 5
    x = torch.randn(T, W, generator=g) * 3
    y = _rnd(g, T, W + 3, dtype=dt)[:, :W]           # a strided view
    w1 = 1.0 + 0.3 * torch.randn(W, generator=g)
    xd = x.clone().to(dev)
    h = hops.norm_residual_add_(xd, y.to(dev), w1.to(dev), 1e-5, dt)
    want = x.to(F64) + o_rms(y.to(F64), 1e-5) * w1.to(F64)
    _close(xd, want, ("x", torch.float32), "residual")
    _close(h, want, target, "operand")


@pytest.mark.parametrize("target", TARGETS)
def test_gelu_gate_and_head_gate(target):
    dev, dt = target
    g = torch.Generator().manual_seed(3)
    z = _rnd(g, 7, 2 * 37, dtype=dt, std=2.0)
    want = o_gelu_tanh(z[:, :37].to(F64)) * z[:, 37:].to(F64)
    _close(hops.gelu_tanh_mul(z.to(dev)), want, target)
    H, Dv = 5, 12
    o = torch.randn(7, H * Dv, generator=g)
    gate = _rnd(g, 7, H + 2, dtype=dt, std=2.0)[:, :H]
    want = (o.to(F64).view(7, H, Dv)
            * o_sigmoid(gate.to(F64))[:, :, None]).reshape(7, H * Dv)
    got = hops.norm_sigmoid_gate(o.to(dev), None, gate.to(dev), 0.0, dt,
                                 gate_cols=Dv)
    _close(got, want, target)


# ---------------------------------- whole-row norm, rotate-half, paged store
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv,rot", [(4, 2, 8, 6, 4), (3, 1, 10, 4, 10),
                                          (2, 2, 6, 6, 0), (8, 4, 64, 32, 16)])
def test_rownorm_rotate_store(target, H, G, D, Dv, rot):
    dev, dt = target
    g = torch.Generator().manual_seed(H * D)
    pos = [0, 1, 7, 300, 40001]
    T = len(pos)
    big = _rnd(g, T, H * D + G * D + G * Dv, dtype=dt)
    q, k = big[:, :H * D], big[:, H * D:H * D + G * D]
    v = big[:, H * D + G * D:]
    qw = (1.0 + 0.2 * torch.randn(H * D, generator=g))
    kw = (1.0 + 0.2 * torch.randn(G * D, generator=g))
    rc = dict(base=50.0, dims=rot)
    inv = torch.tensor([50.0 ** (-2.0 * i / max(rot, 1))
                        for i in range(rot // 2)], dtype=F64)
    slots = [5 * BS + 3, 0, 2 * BS + 15, -1, 7 * BS]
    kc = torch.zeros(9, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(9, G, BS, Dv, dtype=dt, device=dev)
    bd = big.to(dev)
    qo = hops.rownorm_rope_store(
        bd[:, :H * D], bd[:, H * D:H * D + G * D], bd[:, H * D + G * D:],
        qw.to(dev), kw.to(dev), 1e-5, torch.tensor(pos, device=dev),
        inv.to(dev), rot, H, G, kc, vc, torch.tensor(slots, device=dev))
    qn = (o_rms(q.to(F64), 1e-5) * qw.to(F64)).view(T, H, D)
    kn = (o_rms(k.to(F64), 1e-5) * kw.to(F64)).view(T, G, D)
    for t in range(T):
        for a in range(H):
            want = o_rotate_halves(qn[t, a], pos[t], rc) if rot else qn[t, a]
            _close(qo[t].view(H, D)[a], want, target, ("q", t, a), scale=2)
        if slots[t] < 0:
            continue
        b, off = divmod(slots[t], BS)
        for a in range(G):
            want = o_rotate_halves(kn[t, a], pos[t], rc) if rot else kn[t, a]
            _close(kc[b, a, off], want, target, ("k", t, a), scale=2)
            _close(vc[b, a, off], v[t].view(G, Dv)[a].to(F64), target)
    assert float(kc[3].abs().max()) == 0.0          # slot -1 stored nothing


# --------------------------------------------- windowed attention with a sink
def _to_pages(K, V, order, n_blocks, dev):
    kc = torch.zeros(n_blocks, K.shape[1], BS, K.shape[2], dtype=K.dtype)
    vc = torch.zeros(n_blocks, V.shape[1], BS, V.shape[2], dtype=V.dtype)
    for p in range(K.shape[0]):
        kc[order[p // BS], :, p % BS] = K[p]
        vc[order[p // BS], :, p % BS] = V[p]
    return kc.to(dev), vc.to(dev)


def _paged(L, G, D, Dv, dt, dev, g):
    """Random keys/values of one sequence scattered over pages."""
    nb = (L + BS - 1) // BS
    order = torch.randperm(nb + 3, generator=g).tolist()[:nb]
    K, V = _rnd(g, L, G, D, dtype=dt), _rnd(g, L, G, Dv, dtype=dt)
    kc, vc = _to_pages(K, V, order, nb + 3, dev)
    return K, V, kc, vc, order


def _attn_oracle(q, K, V, pos, H, G, scale, window, sink):
    D, Dv = K.shape[-1], V.shape[-1]
    out = torch.zeros(H, Dv, dtype=F64)
    lo = max(0, pos - window + 1) if window else 0
    for a in range(H):
        kv = a // (H // G)
        out[a] = o_attend(q.view(H, D)[a].to(F64), K[lo:pos + 1, kv].to(F64),
                          V[lo:pos + 1, kv].to(F64), scale,
                          None if sink is None else sink[a].to(F64))
    return out


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 8, 6), (3, 1, 24, 10),
                                      (8, 2, 64, 64), (6, 1, 128, 96),
                                      (4, 4, 256, 128)])
def test_standout_key_at_window_edges(target, H, G, D, Dv):
    """One key gets a score far above the rest. When it sits on the last
    position the window still holds, the output is its value; one position
    further back it must not be seen at all. The key is placed so that it
    falls on a page's first and last row and on a 32-key tile border, for
    prompt rows and for single decoded rows."""
    dev, dt = target
    g = torch.Generator().manual_seed(H + D)
    L = 150
    scale = 1.0
    for window in (1, 2, 17, 33, 64, 100):
        K0, V, _, _, order = _paged(L, G, D, Dv, dt, dev, g)
        sink = torch.randn(H, generator=g)
        for pos in (L - 1, 127, 96):
            for dist, seen in ((window - 1, True), (window, False)):
                j = pos - dist
                if j < 0:
                    continue
                # key j is the longest by far and every head's query points
                # along it: no other key can reach its score
                K = K0.clone()
                K[j] = (K[j].float() * 4.0 * K0.float().norm(dim=-1).max()
                        / K[j].float().norm(dim=-1, keepdim=True)).to(dt)
                kc, vc = _to_pages(K, V, order, len(order) + 3, dev)
                q = _rnd(g, H, D, dtype=dt, std=0.05)
                for a in range(H):
                    kj = K[j, a // (H // G)].float()
                    q[a] += (40.0 * kj / kj.norm() ** 2).to(dt)
                want = _attn_oracle(q.reshape(-1), K, V, pos, H, G, scale,
                                    window, sink)
                tables = _i32([order], dev)
                # (a) decoded alone
                out = torch.empty(1, H, Dv, device=dev)
                hops.capped_attn(q.reshape(1, -1).to(dev), kc, vc, tables,
                                 None, _i32([pos + 1], dev), H, scale, 0.0,
                                 out, window=window, sink=sink.to(dev))
                _close(out[0], want, target, (window, pos, dist, "dec"), 3)
                # (b) last row of a prompt portion of 5 rows
                n = min(5, pos + 1)
                qq = torch.cat([_rnd(g, n - 1, H * D, dtype=dt),
                                q.reshape(1, -1)]).to(dev)
                out = torch.empty(n, H, Dv, device=dev)
                hops.capped_attn(qq, kc, vc, tables, _i32([0, n], dev),
                                 _i32([pos + 1], dev), H, scale, 0.0, out,
                                 window=window, sink=sink.to(dev))
                _close(out[-1], want, target, (window, pos, dist, "pre"), 3)
                if seen and window > 1:
                    # the standout key carries nearly all the weight
                    kvj = V[j].to(F64)
                    for a in range(H):
                        d = (want[a] - kvj[a // (H // G)]).abs().max()
                        assert float(d) < 0.2 * float(kvj.abs().max())


@pytest.mark.parametrize("target", TARGETS)
def test_sink_takes_weight_but_no_value(target):
    dev, dt = target
    g = torch.Generator().manual_seed(11)
    H, G, D, Dv, L = 4, 2, 16, 8, 40
    K, V, kc, vc, order = _paged(L, G, D, Dv, dt, dev, g)
    q = _rnd(g, 1, H * D, dtype=dt)
    sink = torch.tensor([-30.0, 0.0, 6.0, 40.0])
    out = torch.empty(1, H, Dv, device=dev)
    hops.capped_attn(q.to(dev), kc, vc, _i32([order], dev), None,
                     _i32([L], dev), H, 0.3, 0.0, out, window=0,
                     sink=sink.to(dev))
    want = _attn_oracle(q[0], K, V, L - 1, H, G, 0.3, 0, sink)
    _close(out[0], want, target, "sink", 3)
    no = torch.empty(1, H, Dv, device=dev)
    hops.capped_attn(q.to(dev), kc, vc, _i32([order], dev), None,
                     _i32([L], dev), H, 0.3, 0.0, no)
    # a very negative sink changes nothing; a dominant one empties the head
    _close(out[0, 0], no[0, 0].cpu(), target, "no sink", 3)
    assert float(out[0, 3].abs().max()) < 1e-6


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv,window", [(4, 2, 8, 6, 0), (6, 2, 64, 32, 40),
                                             (16, 4, 128, 128, 300),
                                             (2, 1, 40, 24, 9)])
def test_batch_of_unequal_requests_on_scattered_pages(target, H, G, D, Dv,
                                                      window):
    """Prompt portions of several requests in one call and their decoded
    rows in another, every request on its own scattered pages; a far key
    stands out for one of them."""
    dev, dt = target
    g = torch.Generator().manual_seed(window + D)
    seqs = [(0, 70), (290, 3), (500, 1), (33, 64), (15, 2)]     # (ctx, new)
    n_blocks = sum((c + n + BS - 1) // BS for c, n in seqs) + 5
    perm = torch.randperm(n_blocks, generator=g).tolist()
    kc = torch.zeros(n_blocks, G, BS, D, dtype=dt)
    vc = torch.zeros(n_blocks, G, BS, Dv, dtype=dt)
    Ks, Vs, tables, at = [], [], [], 0
    for c, n in seqs:
        L = c + n
        nb = (L + BS - 1) // BS
        order = perm[at:at + nb]
        at += nb
        K, V = _rnd(g, L, G, D, dtype=dt), _rnd(g, L, G, Dv, dtype=dt)
        for p in range(L):
            kc[order[p // BS], :, p % BS] = K[p]
            vc[order[p // BS], :, p % BS] = V[p]
        Ks.append(K); Vs.append(V); tables.append(order)
    width = max(len(t) for t in tables)
    tb = _i32([t + [0] * (width - len(t)) for t in tables], dev)
    kc, vc = kc.to(dev), vc.to(dev)
    sink = torch.randn(H, generator=g)
    T = sum(n for _, n in seqs)
    q = _rnd(g, T, H * D, dtype=dt, std=0.5)
    # request 2 (one row at position 500): key 3 stands out (far back)
    row2 = seqs[0][1] + seqs[1][1]
    for a in range(H):
        kk = Ks[2][3, a // (H // G)].float()
        q[row2, a * D:(a + 1) * D] = (30.0 * kk / kk.norm() ** 2).to(dt)
    scale = 1.0
    cu = [0]
    for _, n in seqs:
        cu.append(cu[-1] + n)
    out = torch.empty(T, H, Dv, device=dev)
    hops.capped_attn(q.to(dev), kc, vc, tb, _i32(cu, dev),
                     _i32([c + n for c, n in seqs], dev), H, scale, 0.0, out,
                     window=window, sink=sink.to(dev))
    for s, (c, n) in enumerate(seqs):
        for i in range(n):
            want = _attn_oracle(q[cu[s] + i], Ks[s], Vs[s], c + i, H, G,
                                scale, window, sink)
            _close(out[cu[s] + i], want, target, (s, i), 3)
    # the last row of every request once more, as decoded rows
    last = [cu[s + 1] - 1 for s in range(len(seqs))]
    out2 = torch.empty(len(seqs), H, Dv, device=dev)
    hops.capped_attn(q[last].to(dev), kc, vc, tb, None,
                     _i32([c + n for c, n in seqs], dev), H, scale, 0.0, out2,
                     window=window, sink=sink.to(dev))
    _close(out2, out[last].cpu(), target, "decode rows", 3)


# ------------------------------------------- latent attention, no positions
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,r", [(2, 12), (4, 64), (3, 40), (16, 128)])
def test_latent_rows_without_rotated_part(target, H, r):
    """The cached row is the normed latent alone (no rotated tail). Queries
    already folded through the key up-projection are scored against the
    rows; a key far back, on a page's last row, stands out for one query."""
    dev, dt = target
    g = torch.Generator().manual_seed(H * r)
    L, n = 200, 6                          # context rows, then a portion of 6
    raw = _rnd(g, L, r, dtype=dt)
    w = 1.0 + 0.2 * torch.randn(r, generator=g)
    nb = (L + BS - 1) // BS
    order = torch.randperm(nb + 2, generator=g).tolist()[:nb]
    cache = torch.zeros(nb + 2, BS, r, dtype=dt, device=dev)
    slots = torch.tensor([order[p // BS] * BS + p % BS for p in range(L)])
    none = torch.zeros(0, dtype=F64, device=dev)
    hops.latent_kv_store(raw.to(dev), w.to(dev), 1e-5,
                         torch.arange(L, device=dev), none, 1.0, 0, cache,
                         slots.to(dev), r)
    c = o_rms(raw.to(F64), 1e-5) * w.to(F64)
    got_rows = cache.view(-1, r)[slots.to(dev)]
    _close(got_rows, c, target, "rows", 2)
    c = got_rows.cpu().to(F64)             # what the kernel reads
    q = _rnd(g, n, H, r, dtype=dt, std=0.3)
    far = 15                               # last row of the first page
    q[n - 1] = (25.0 * c[far] / c[far].norm() ** 2).to(dt)
    out = torch.empty(n, H, r, device=dev)
    hops.latent_attn(q.to(dev), cache, _i32([order], dev), _i32([0, n], dev),
                     _i32([L], dev), 0.8, r, out)
    for i in range(n):
        pos = L - n + i
        for a in range(H):
            want = o_attend(q[i, a].to(F64), c[:pos + 1], c[:pos + 1], 0.8)
            _close(out[i, a], want, target, (i, a), 3)
    assert float((out[n - 1, 0].cpu().to(F64) - c[far]).abs().max()) \
        < 0.2 * float(c[far].abs().max())
    # the last row once more as a decoded row
    out2 = torch.empty(1, H, r, device=dev)
    hops.latent_attn(q[n - 1:].to(dev), cache, _i32([order], dev), None,
                     _i32([L], dev), 0.8, r, out2)
    _close(out2[0], out[n - 1].cpu(), target, "decode row", 3)


# ------------------------------------------------------------ the delta rule
def _delta_inputs(g, T, H, G, D, Dv, dt):
    return (_rnd(g, T, G * D, dtype=dt), _rnd(g, T, G * D, dtype=dt),
            _rnd(g, T, H * Dv, dtype=dt), _rnd(g, T, H, dtype=dt, std=2.0),
            _rnd(g, T, H, dtype=dt, std=2.0))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 6, 5), (1, 1, 16, 16),
                                      (3, 3, 40, 12), (4, 2, 64, 64),
                                      (2, 1, 256, 32), (32, 8, 32, 64)])
def test_delta_rule_through_portions_and_slots(target, H, G, D, Dv):
    """A sequence fed in portions (down to one and two tokens, through the
    prompt kernel and the single-row kernel) must give what the whole gives;
    its slot held another sequence's state before; a row without a slot
    runs from zero and stores nothing."""
    dev, dt = target
    g = torch.Generator().manual_seed(H * D + Dv)
    T = 45
    q, k, v, b, a = _delta_inputs(g, T, H, G, D, Dv, dt)
    A_log = torch.randn(H, generator=g) * 0.5 - 1.0
    dt_bias = torch.randn(H, generator=g)
    want, S_end = o_delta_core(
        q.to(F64).view(T, G, D), k.to(F64).view(T, G, D),
        v.to(F64).view(T, H, Dv), b.to(F64), a.to(F64), A_log.to(F64),
        dt_bias.to(F64))
    dq, dk, dv, db, da = (x.to(dev) for x in (q, k, v, b, a))
    for cuts in ([T], [1, 2, 17, 1, 1, 16, 7], [2] * 5 + [33, 1, 1]):
        state = torch.randn(3, H, D, Dv, generator=g).to(dev)   # stale
        before = state.clone()
        out = torch.empty(T, H, Dv, device=dev)
        at = 0
        for n in cuts:
            rows = slice(at, at + n)
            single = n == 1 and at > 0
            # a second request without a slot rides along in prompt steps
            if single:
                slots, cu, ctx = [1], None, [at]
                sel = rows
                o = out[rows]
            else:
                slots, cu, ctx = [1, -1], [0, n, n + 2], [at, 5]
                sel = list(range(at, at + n)) + [0, 1]
                o = torch.empty(n + 2, H, Dv, device=dev)
            hops.delta_rule(dq[sel], dk[sel], dv[sel], db[sel], da[sel],
                            dt_bias.to(dev), A_log.to(dev), state,
                            _i32(slots, dev), None if cu is None
                            else _i32(cu, dev), _i32(ctx, dev), G, o)
            if not single:
                out[rows] = o[:n]
            at += n
        _close(out, want, target, cuts, 5)
        _close(state[1], S_end, target, ("state", cuts), 5)
        assert torch.equal(state[0], before[0]) and \
            torch.equal(state[2], before[2])


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv", [(2, 1, 40, 12), (4, 2, 64, 64),
                                      (2, 2, 128, 128), (3, 1, 16, 100)])
def test_delta_rule_long_chunks(target, H, G, D, Dv):
    """Chunks long enough for the piece-parallel passes (pieces of 128
    tokens, the last one short), from a zero state and from a carried one,
    beside a short request in the same call."""
    dev, dt = target
    g = torch.Generator().manual_seed(D + Dv)
    T = 650
    q, k, v, b, a = _delta_inputs(g, T, H, G, D, Dv, dt)
    A_log = torch.randn(H, generator=g) * 0.5 - 2.0
    dt_bias = torch.randn(H, generator=g)
    want, S_end = o_delta_core(
        q.to(F64).view(T, G, D), k.to(F64).view(T, G, D),
        v.to(F64).view(T, H, Dv), b.to(F64), a.to(F64), A_log.to(F64),
        dt_bias.to(F64))
    dq, dk, dv, db, da = (x.to(dev) for x in (q, k, v, b, a))
    for cuts in ([T], [37, T - 37]):
        state = torch.randn(3, H, D, Dv, generator=g).to(dev)   # stale
        out = torch.empty(T, H, Dv, device=dev)
        at = 0
        for n in cuts:
            # the short request (rows 0..4 again, no slot) comes first
            sel = list(range(5)) + list(range(at, at + n))
            o = torch.empty(n + 5, H, Dv, device=dev)
            hops.delta_rule(dq[sel], dk[sel], dv[sel], db[sel], da[sel],
                            dt_bias.to(dev), A_log.to(dev), state,
                            _i32([-1, 2], dev), _i32([0, 5, n + 5], dev),
                            _i32([0, at], dev), G, o, max_q_len=n)
            out[at:at + n] = o[5:]
            _close(o[:5], want[:5], target, ("short", cuts), 5)
            at += n
        _close(out, want, target, cuts, 10)
        _close(state[2], S_end, target, ("state", cuts), 10)


@pytest.mark.parametrize("target", TARGETS)
def test_delta_rule_long_decoding_batch(target):
    """Four sequences decode 120 tokens each, one row per sequence and call
    (the whole-state kernel), after prompts of unequal length."""
    dev, dt = target
    g = torch.Generator().manual_seed(5)
    H, G, D, Dv = 4, 2, 32, 16
    A_log = torch.randn(H, generator=g) * 0.5 - 1.5
    dt_bias = torch.randn(H, generator=g)
    lens = [7, 1, 30, 16]
    n_dec = 120
    data = [_delta_inputs(g, L + n_dec, H, G, D, Dv, dt) for L in lens]
    want = [o_delta_core(d[0].to(F64).view(-1, G, D),
                         d[1].to(F64).view(-1, G, D),
                         d[2].to(F64).view(-1, H, Dv), d[3].to(F64),
                         d[4].to(F64), A_log.to(F64), dt_bias.to(F64))[0]
            for d in data]
    state = torch.randn(4, H, D, Dv, generator=g).to(dev)
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    cat = [torch.cat([d[i][:L] for d, L in zip(data, lens)]).to(dev)
           for i in range(5)]
    out = torch.empty(cu[-1], H, Dv, device=dev)
    slots = _i32([2, 0, 3, 1], dev)
    hops.delta_rule(*cat, dt_bias.to(dev), A_log.to(dev), state, slots,
                    _i32(cu, dev), _i32([0] * 4, dev), G, out)
    for s, L in enumerate(lens):
        _close(out[cu[s]:cu[s + 1]], want[s][:L], target, ("prompt", s), 5)
    for t in range(n_dec):
        rows = [torch.stack([d[i][L + t] for d, L in zip(data, lens)]).to(dev)
                for i in range(5)]
        o = torch.empty(4, H, Dv, device=dev)
        hops.delta_rule(*rows, dt_bias.to(dev), A_log.to(dev), state, slots,
                        None, _i32([L + t for L in lens], dev), G, o)
        if t % 17 == 0 or t == n_dec - 1:
            for s, L in enumerate(lens):
                _close(o[s], want[s][L + t], target, ("decode", s, t), 10)


@pytest.mark.parametrize("target", TARGETS)
def test_delta_rule_overwrites_what_a_key_held(target):
    """With beta = 1 and no decay, writing (k, v2) after (k, v1) leaves v2
    alone under k: the read-out with q = k is v2 / sqrt(D), not the sum."""
    dev, dt = target
    H = G = 1
    D, Dv = 8, 4
    k = torch.zeros(2, D); k[:, 2] = 3.0
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-5.0, 6.0, 0.5, 8.0]])
    b = torch.full((2, 1), 40.0)           # sigmoid -> 1
    a = torch.full((2, 1), -40.0)          # softplus -> 0, decay -> 1
    args = [x.to(dt).to(dev) for x in (k, k, v, b, a)]
    state = torch.zeros(1, H, D, Dv, device=dev)
    out = torch.empty(2, H, Dv, device=dev)
    hops.delta_rule(*args, torch.zeros(1, device=dev),
                    torch.zeros(1, device=dev), state, _i32([0], dev),
                    _i32([0, 2], dev), _i32([0], dev), G, out)
    _close(out[1, 0], v[1].to(F64) / math.sqrt(D), target, "overwrite", 5)
    _close(out[0, 0], v[0].to(F64) / math.sqrt(D), target, "first", 5)
