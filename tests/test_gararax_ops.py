"""The mechanisms of the Gararax decoder one at a time: the op layer
(xllm_service_amd.ops.hybrid; fp32 torch on the CPU, HIP kernels under the gpu
marker, fp32 and bf16 storage) against the plain functions of
tests/gararax_oracle.py. Inputs are made so that a fault shows: one key whose
score stands out just inside or just outside the window or the kept first
keys, at page and tile borders, or far back; a sink that takes most of the
weight; corrections that make choice scores negative."""
import math

import pytest
import torch

import gararax_oracle as go
from xllm_service_amd.models.mixers import banded_rope_frequencies
from xllm_service_amd.models.moe import RoutedExperts
from xllm_service_amd.ops import hybrid as hops

F64 = torch.float64
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
    same inputs as the fp64 functions)."""
    return (torch.randn(*shape, generator=g) * std).bfloat16().to(dtype)


def _i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


# ------------------------------------------------------- norms and gates
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("W", [20, 257, 1288])
@pytest.mark.parametrize("y32", [False, True])
def test_post_norm_add_with_next_norm(target, W, y32):
    dev, dt = target
    g = torch.Generator().manual_seed(W)
    T = 5
    x = torch.randn(T, W, generator=g) * 3
    y = _rnd(g, T, W + 3, dtype=torch.float32 if y32 else dt)[:, :W]
    w1 = 0.3 * (1.0 + 0.3 * torch.randn(W, generator=g))
    wn = 1.0 + 0.3 * torch.randn(W, generator=g)
    want = x.to(F64) + go.rms_unit(y.to(F64), 1e-5) * w1.to(F64)
    xd = x.clone().to(dev)
    h = hops.norm_residual_add_(xd, y.to(dev), w1.to(dev), 1e-5, dt,
                                wn.to(dev))
    _close(xd, want, ("x", torch.float32), "residual")
    _close(h, go.rms_norm(want, wn.to(F64), 1e-5), target, "next input")
    xd = x.clone().to(dev)
    h = hops.norm_residual_add_(xd, y.to(dev), w1.to(dev), 1e-5, dt)
    _close(h, want, target, "plain operand")


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("F", [1, 37, 256, 1500])
def test_polynorm(target, F):
    dev, dt = target
    g = torch.Generator().manual_seed(F)
    z = _rnd(g, 6, F + 5, dtype=dt, std=1.7)[:, :F]       # a strided view
    for coef in ([0.5, -0.8, 0.3, 0.2], [0.0, 1.0, 0.0, 0.0],
                 [0.0, 0.0, 1.0, -1.0]):
        c = torch.tensor(coef)
        got = hops.polynorm(z.to(dev), c.to(dev), 1e-5)
        _close(got, go.polynorm(z.to(F64), c.to(F64), 1e-5), target, coef)


@pytest.mark.parametrize("target", TARGETS)
def test_gelu_gate_of_two_tensors(target):
    dev, dt = target
    g = torch.Generator().manual_seed(3)
    a = _rnd(g, 7, 11, dtype=dt, std=2.0)
    table = _rnd(g, 7, 40, dtype=dt)
    u = table[:, 22:33]                                  # a layer's part
    got = hops.gelu_tanh_gate(a.to(dev), u.to(dev))
    _close(got, go.gelu_tanh(a.to(F64)) * u.to(F64), target)


# ------------------------------------------------ rotary frequencies, turns
def test_banded_frequencies_cover_all_three_bands():
    rot = dict(base=10000.0, dims=32,
               scaling=dict(factor=8.0, low=1.0, high=4.0, original=256))
    f0 = go.rotary_frequencies(dict(base=10000.0, dims=32))
    want = go.rotary_frequencies(rot)
    kept = (want == f0).sum()
    divided = torch.isclose(want, f0 / 8.0, rtol=1e-12).sum()
    assert kept > 0 and divided > 0 and kept + divided < 16
    assert torch.allclose(banded_rope_frequencies(rot), want, rtol=1e-12)
    plain = dict(base=77.0, dims=6)
    assert torch.allclose(banded_rope_frequencies(plain),
                          go.rotary_frequencies(plain), rtol=1e-12)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("pairs", [True, False])
@pytest.mark.parametrize("H,G,D,Dv,rot,unit", [
    (4, 2, 8, 6, 4, True), (3, 1, 10, 4, 10, False), (2, 2, 6, 6, 0, True),
    (8, 4, 64, 32, 16, True), (2, 1, 128, 80, 64, False),
    (1, 1, 200, 8, 200, True)])
def test_turn_unit_norm_and_paged_store(target, pairs, H, G, D, Dv, rot, unit):
    dev, dt = target
    g = torch.Generator().manual_seed(H * D + rot)
    T, nb = 9, 6
    proj = _rnd(g, T, H * D + G * D + G * Dv + 3, dtype=dt)
    q, k = proj[:, :H * D], proj[:, H * D:H * D + G * D]
    v = proj[:, H * D + G * D:H * D + G * D + G * Dv]
    pos = torch.tensor([0, 1, 2, 15, 16, 17, 300, 4097, 70000])
    inv = go.rotary_frequencies(dict(base=50.0, dims=rot)) if rot \
        else torch.zeros(0, dtype=F64)
    slots = torch.tensor([5, 0, 17, -1, 31, 32, 95, 48, 63])
    kc = torch.zeros(nb, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(nb, G, BS, Dv, dtype=dt, device=dev)
    qn = hops.rope_headnorm_store(
        q.to(dev), k.to(dev), v.to(dev), pos.to(dev), inv.to(dev), rot, pairs,
        unit, 1e-5, H, G, kc, vc, slots.to(dev))
    lay = "pairs" if pairs else "halves"

    def prep(z, n):
        z = go.rotate(z.to(F64).view(T, n, D), pos, inv, rot, lay)
        return go.rms_unit(z, 1e-5) if unit else z
    _close(qn.view(T, H, D), prep(q, H), target, "q")
    kw = prep(k, G)
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        _close(kc[s // BS, :, s % BS], kw[t], target, ("k", t))
        _close(vc[s // BS, :, s % BS], v[t].view(G, Dv), target, ("v", t))
    # slot -1 wrote nothing: page 0 row 1..4 and others stay zero except used
    used = {int(s) for s in slots if s >= 0}
    for s in range(nb * BS):
        if s not in used:
            assert float(kc[s // BS, :, s % BS].abs().sum()) == 0.0
    # keys read as values: no value rows, one cache
    kc2 = torch.zeros(nb, G, BS, D, dtype=dt, device=dev)
    hops.rope_headnorm_store(q.to(dev), k.to(dev), None, pos.to(dev),
                             inv.to(dev), rot, pairs, unit, 1e-5, H, G, kc2,
                             kc2, slots.to(dev))
    assert torch.equal(kc2, kc)


# ----------------------------------------------------------- attention
def _paged(k, v, dev, dt, seed, spare=3):
    """Scatter [L, G, D] keys / values over shuffled pages; returns caches
    and the block table row."""
    L, G, D = k.shape
    Dv = v.shape[-1]
    nblk = (L + BS - 1) // BS
    g = torch.Generator().manual_seed(seed)
    order = torch.randperm(nblk + spare, generator=g)[:nblk]
    kc = torch.randn(nblk + spare, G, BS, D, generator=g).to(dt)   # stale data
    vc = torch.randn(nblk + spare, G, BS, Dv, generator=g).to(dt)
    for j in range(L):
        kc[order[j // BS], :, j % BS] = k[j].to(dt)
        vc[order[j // BS], :, j % BS] = v[j].to(dt)
    return kc.to(dev), vc.to(dev), order.to(torch.int32)


def _attn_case(target, H, G, D, Dv, L, n_q, window, keep, standout, seed,
               sink=False, temp=False, same=False, decode=False):
    """The last n_q positions of an L-token sequence ask; key `standout` gets
    a score far above the rest for every query."""
    dev, dt = target
    g = torch.Generator().manual_seed(seed)
    q = _rnd(g, L, H, D, std=0.5)
    k = _rnd(g, L, G, D, std=0.5)
    v = k if same else _rnd(g, L, G, Dv)
    if standout is not None:
        k[standout] = 0.0
        k[standout, :, 0] = 8.0
        q[:, :, 0] = 4.0
    scale = 1.0 / math.sqrt(D)
    hs = (1.0 + 0.5 * torch.rand(H, generator=g)).bfloat16().float() \
        if temp else None
    mask = go.visible(L, window if window else None, keep)
    want = go.attend(q.to(F64), k.to(F64), v.to(F64), scale, mask,
                     head_scale=None if hs is None else hs.to(F64),
                     sink=sink)[L - n_q:]
    kc, vc, table = _paged(k, v, dev, dt, seed)
    if same:
        vc = kc
    out = torch.empty(n_q, H, v.shape[-1], dtype=torch.float32, device=dev)
    qq = q[L - n_q:].reshape(n_q, H * D).to(dt).to(dev)
    sk = torch.zeros(H, device=dev) if sink else None
    hsd = hs.to(dev) if temp else None
    if decode:
        for i in range(n_q):           # each as a decode row of its own length
            hops.capped_attn(qq[i:i + 1], kc, vc, table[None].to(dev), None,
                             _i32([L - n_q + i + 1], dev), H, scale, 0.0,
                             out[i:i + 1], window=window, sink=sk,
                             keep_first=keep, head_scale=hsd)
    else:
        hops.capped_attn(qq, kc, vc, table[None].to(dev), _i32([0, n_q], dev),
                         _i32([L], dev), H, scale, 0.0, out, window=window,
                         sink=sk, keep_first=keep, head_scale=hsd)
    return out, want


SHAPES = [(4, 2, 8, 6), (6, 2, 64, 64), (4, 1, 128, 48), (2, 2, 64, 72),
          (3, 3, 10, 10)]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("H,G,D,Dv", SHAPES)
def test_window_edges_and_kept_first_keys(target, decode, H, G, D, Dv):
    """A standout key just inside / just outside the window of the last
    query, and just inside / just outside the kept first keys."""
    L, n_q, window, keep = 150, 3, 40, 5
    last = L - 1
    for standout in (last - window + 1,      # the oldest key the last sees
                     last - window,          # just out for the last query
                     last - window - 2,      # out for all three
                     keep - 1, keep,         # kept / not kept
                     0, last):
        got, want = _attn_case(target, H, G, D, Dv, L, n_q, window, keep,
                               standout, 100 + standout, decode=decode)
        _close(got, want, target, (standout, decode))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("window,keep", [(1, 0), (1, 3), (16, 16), (17, 15),
                                         (32, 33), (33, 1), (64, 70),
                                         (500, 4), (0, 0)])
def test_windows_at_page_and_tile_borders(target, decode, window, keep):
    for L in (1, 2, 16, 17, 33, 100):
        n_q = min(L, 3)
        got, want = _attn_case(target, 4, 2, 64, 64, L, n_q, window, keep,
                               None, L + window, decode=decode)
        _close(got, want, target, (L, window, keep))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("H,G,D,Dv", SHAPES[:3])
def test_far_key_long_context_decode_partitions(target, H, G, D, Dv,
                                                monkeypatch):
    """A standout key hundreds of positions back: seen without a window,
    unseen with one unless it is a kept first key; the decode context is
    split over several workgroups."""
    monkeypatch.setenv("XLLM_CAPPED_PARTS", "5")
    L = 900
    for window, keep, standout in ((0, 0, 3), (64, 8, 3), (64, 2, 3),
                                   (64, 40, 37), (300, 70, 65)):
        for decode in (True, False):
            got, want = _attn_case(target, H, G, D, Dv, L, 2, window, keep,
                                   standout, L + window, decode=decode)
            _close(got, want, target, (window, keep, standout, decode))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("decode", [False, True])
def test_zero_sink_keys_as_values_and_head_multiplier(target, decode):
    # small scores: the sink's weight 1 / (1 + sum) is most of the mass
    got, want = _attn_case(target, 4, 2, 64, 64, 5, 5, 3, 1, None, 7,
                           sink=True, same=True, decode=decode)
    assert float(want.abs().max()) > 0
    _close(got, want, target, "sink")
    g2, w2 = _attn_case(target, 4, 2, 64, 64, 5, 5, 3, 1, None, 7, same=True,
                        decode=decode)
    assert float((w2 - want).abs().max()) > 0.05      # the sink matters
    got, want = _attn_case(target, 4, 1, 128, 48, 70, 4, 0, 0, None, 8,
                           temp=True, decode=decode)
    _close(got, want, target, "multiplier")
    got, want = _attn_case(target, 3, 3, 10, 10, 40, 4, 9, 2, 31, 9,
                           sink=True, temp=True, same=True, decode=decode)
    _close(got, want, target, "all")


@pytest.mark.parametrize("target", TARGETS)
def test_batch_of_unequal_chunks(target):
    """Three sequences in one prefill call and in one decode call: chunks of
    unequal length with unequal contexts, each against itself alone."""
    dev, dt = target
    H, G, D, Dv, window, keep = 4, 2, 64, 32, 20, 3
    g = torch.Generator().manual_seed(5)
    lens, chunks = [70, 5, 33], [7, 5, 1]
    qs, tabs, wants, caches = [], [], [], []
    nb = sum((L + BS - 1) // BS for L in lens)
    kc = torch.zeros(nb, G, BS, D, dtype=dt)
    vc = torch.zeros(nb, G, BS, Dv, dtype=dt)
    base = 0
    for L, n in zip(lens, chunks):
        q, k, v = _rnd(g, L, H, D), _rnd(g, L, G, D), _rnd(g, L, G, Dv)
        wants.append(go.attend(q.to(F64), k.to(F64), v.to(F64), 0.2,
                               go.visible(L, window, keep))[L - n:])
        nblk = (L + BS - 1) // BS
        for j in range(L):
            kc[base + j // BS, :, j % BS] = k[j].to(dt)
            vc[base + j // BS, :, j % BS] = v[j].to(dt)
        tabs.append(list(range(base, base + nblk)))
        base += nblk
        qs.append(q[L - n:].reshape(n, H * D))
    width = max(len(t) for t in tabs)
    table = _i32([t + [0] * (width - len(t)) for t in tabs], dev)
    qq = torch.cat(qs).to(dt).to(dev)
    out = torch.empty(sum(chunks), H, Dv, dtype=torch.float32, device=dev)
    cu = [0, 7, 12, 13]
    hops.capped_attn(qq, kc.to(dev), vc.to(dev), table, _i32(cu, dev),
                     _i32(lens, dev), H, 0.2, 0.0, out, window=window,
                     keep_first=keep)
    _close(out, torch.cat(wants), target, "prefill batch")
    last = torch.cat([q[-1:] for q in qs]).to(dt).to(dev)
    out = torch.empty(3, H, Dv, dtype=torch.float32, device=dev)
    hops.capped_attn(last, kc.to(dev), vc.to(dev), table, None,
                     _i32(lens, dev), H, 0.2, 0.0, out, window=window,
                     keep_first=keep)
    _close(out, torch.stack([w[-1] for w in wants]), target, "decode batch")


# -------------------------------------------------------------- experts
def _route_case(g, T, W, experts, identity, top, groups, corr_scale):
    r = dict(experts=experts, top=top, identity=identity)
    if groups:
        r["groups"] = dict(count=groups[0], keep=groups[1])
    n = experts + identity
    w = {"router": _rnd(g, n, W, std=2.0 / math.sqrt(W)),
         "correction": _rnd(g, n, std=corr_scale)}
    return r, w


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("experts,identity,top,groups,corr", [
    (10, 2, 3, (4, 2), 0.05), (6, 0, 2, None, 0.0), (5, 1, 1, (3, 1), 0.3),
    (16, 0, 3, (4, 1), 2.0), (64, 8, 6, (8, 4), 0.01), (3, 0, 3, None, 0.1)])
def test_router(target, experts, identity, top, groups, corr):
    """Softmax scores, choice on score + correction (strongly negative
    corrections included: a masked group must lose to them), groups scored
    by their best member, weights renormalised."""
    dev, dt = target
    g = torch.Generator().manual_seed(experts + top)
    T, W = 64, 32
    r, w = _route_case(g, T, W, experts, identity, top, groups, corr)
    if corr >= 2.0:
        w["correction"] = -w["correction"].abs() - 1.0      # all negative
    h = _rnd(g, T, W, dtype=dt)
    ids_w, wt_w = go.route(h.to(F64), {k: v.to(F64) for k, v in w.items()},
                           "", r)
    ids, wts = hops.moe_route(
        h.to(dev), w["router"].to(dev), top, groups[0] if groups else 1,
        groups[1] if groups else 1, softmax=True,
        correction=w["correction"].to(dev), group_max=True, normalize=True)
    # a near tie may be cut either way: compare the sets row by row
    same = [set(a) == set(b) for a, b in zip(ids.cpu().tolist(),
                                             ids_w.tolist())]
    assert sum(same) >= T - 2, sum(same)
    for t in range(T):
        if same[t]:
            a = dict(zip(ids[t].cpu().tolist(), wts[t].cpu().tolist()))
            for j, x in zip(ids_w[t].tolist(), wt_w[t].tolist()):
                assert abs(a[j] - x) < 1e-4, (t, j)
    assert float((wts.sum(-1) - 1).abs().max()) < 1e-5


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("T", [3, 70, 300])
@pytest.mark.parametrize("identity,shared,groups", [(2, 5, (3, 2)),
                                                    (0, 0, None), (4, 0, (2, 1))])
def test_expert_layer_every_execution_shape(target, T, identity, shared,
                                            groups):
    """The layer with identity and shared experts against the plain sum; the
    dense, padded and expert-by-expert shapes give the same result."""
    dev, dt = target
    W, ff, experts, top = 24, 10, 4, 2
    cfg = go.make_config(width=W, layers=[go.attn(mlp=go.moe(
        ff=ff, experts=experts, top=top, identity=identity, groups=groups,
        shared=shared))])
    w = go.make_weights(cfg, seed=T)
    mlp = cfg["layers"][0]["mlp"]
    g = torch.Generator().manual_seed(T)
    h = _rnd(g, T, W, dtype=dt)
    if T == 300:                         # uneven load: one expert for most
        h[: 2 * T // 3] = h[0] + 0.01 * h[: 2 * T // 3]
        h = h.bfloat16().to(dt)
    want = go.ff_moe(h.to(F64), {k: v.to(F64) for k, v in w.items()},
                     "l0.mlp.", mlp, 1e-5)
    m = RoutedExperts(W, ff, experts, top, groups[0] if groups else 1,
                      groups[1] if groups else 1, dt, identity=identity,
                      softmax=True, correction=True, group_max=True,
                      normalize=True, shared_ff=shared)
    with torch.no_grad():
        m.router.copy_(w["l0.mlp.router"])
        m.correction.copy_(w["l0.mlp.correction"])
        for j in range(experts):
            m.w_gate_up[j].copy_(torch.cat([w[f"l0.mlp.e{j}.gate"],
                                            w[f"l0.mlp.e{j}.up"]]))
            m.w_down[j].copy_(w[f"l0.mlp.e{j}.down"])
        if shared:
            m.shared_gate_up.copy_(torch.cat([w["l0.mlp.shared.gate"],
                                              w["l0.mlp.shared.up"]]))
            m.shared_down.copy_(w["l0.mlp.shared.down"])
    m = m.to(dev)
    with torch.no_grad():
        got = m(h.to(dev))
        m.dense_max_tokens = 0 if T <= 64 else 10 ** 6     # the other shape
        again = m(h.to(dev))
    bad = go.rel_err(got.cpu(), want) > (1e-4 if dt == torch.float32 else 0.1)
    assert int(bad.sum()) <= 1 + T // 50, int(bad.sum())   # near-tie rows
    assert float(go.rel_err(again.cpu(), got.cpu()).median()) < \
        (1e-5 if dt == torch.float32 else 2e-2)


@pytest.mark.parametrize("target", TARGETS)
def test_combine_with_identity_rows_and_added_output(target):
    dev, dt = target
    g = torch.Generator().manual_seed(11)
    T, W, top = 9, 40, 3
    y = _rnd(g, 20, W, dtype=dt)
    ident = _rnd(g, T, W + 4, dtype=dt)[:, :W]
    extra = _rnd(g, T, W, dtype=dt)
    rows = torch.randint(-1, 20, (T, top), generator=g).to(torch.int32)
    rows[0] = -1
    wts = torch.rand(T, top, generator=g)
    src = torch.where((rows < 0)[:, :, None], ident.to(F64)[:, None, :],
                      y.to(F64)[rows.clamp(min=0).long()])
    want = (src * wts.to(F64)[:, :, None]).sum(1) + extra.to(F64)
    got = hops.moe_combine(y.to(dev), rows.to(dev), wts.to(dev), T,
                           ident.to(dev), extra.to(dev))
    _close(got, want, ("", torch.float32), "combine")
