"""Pure-PyTorch fp32 reference implementations of every HIP op.

These serve two purposes:
  * numerics oracles for the GPU kernels (tests/test_gpu_ops.py compares the
    HIP kernels against these at fp32)
  * the CPU execution path (OPT-125m control-plane config)

They are intentionally simple and readable, not fast.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


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


def norm_sigmoid_gate(o, w, gate, eps, out_dtype, gate_cols=1):
    """rmsnorm(o) * w * sigmoid(gate); w None skips the norm. gate_cols > 1:
    one gate entry serves that many neighbouring columns of o."""
    z = o.float()
    if w is not None:
        z = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    g = torch.sigmoid(gate.float())
    if gate_cols > 1:
        g = g.repeat_interleave(gate_cols, -1)
    return (z * g).to(out_dtype)


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


def moe_route(h, w_router, top, n_groups, keep, softmax=False,
              correction=None, group_max=False, normalize=False):
    """Top-k routing with group limiting. Scores: sigmoid of the fp32 logits,
    or their softmax over all experts. The choice is made on the scores plus
    `correction` (when given); the weights are the plain scores of the
    chosen, divided by their sum (+ 1e-20) with `normalize`. Experts form
    n_groups equal neighbouring groups, scored by the sum of their two
    largest choice scores (by the largest one with `group_max`); only the
    best `keep` groups are eligible. Returns (ids [T, top] int32, weights
    [T, top] fp32)."""
    z = h.float() @ w_router.float().T
    s = torch.softmax(z, -1) if softmax else torch.sigmoid(z)
    T, E = s.shape
    sm = s if correction is None else s + correction.float()
    if n_groups > 1:
        sg = sm.view(T, n_groups, E // n_groups)
        if group_max:
            gs = sg.max(-1).values
        else:
            gs = sg.topk(min(2, E // n_groups), -1).values.sum(-1)
        best = gs.topk(keep, -1).indices
        gm = torch.zeros_like(gs, dtype=torch.bool).scatter(1, best, True)
        sm = sg.masked_fill(~gm[:, :, None], float("-inf")).reshape(T, E)
    idx = sm.topk(top, -1).indices
    wts = s.gather(1, idx)
    if normalize:
        wts = wts / (wts.sum(-1, keepdim=True) + 1e-20)
    return idx.to(torch.int32), wts


def silu_mul(x):
    """[..., 2F] -> silu(x[..., :F]) * x[..., F:], dtype preserved."""
    return silu_and_mul(x)


# ---------------------------------------------------------------------------
# Residual streams, short convolutions with state, data-dependent linear
# recurrences, soft-capped paged attention. fp32 throughout.
# ---------------------------------------------------------------------------
def streams_mix_norm(x, w_in, g, b, eps, out_dtype):
    """x fp32 [T, S, W] -> layer norm of sum_s w_in[s] x[:, s], times g
    plus b, [T, W]. w_in None: plain sum."""
    u = x.sum(1) if w_in is None else torch.einsum("tsw,s->tw", x, w_in)
    mu = u.mean(-1, keepdim=True)
    var = (u - mu).pow(2).mean(-1, keepdim=True)
    return ((u - mu) * torch.rsqrt(var + eps) * g + b).to(out_dtype)


def streams_update(x, mix, w_out, y1, a1, y2, a2):
    """x[:, j] <- sum_s mix[s, j] x[:, s] + w_out[j] (a1 y1 + a2 y2)."""
    S = x.shape[1]
    y = a1 * y1.float()
    if y2 is not None:
        y = y + a2 * y2.float()
    m = torch.eye(S) if mix is None else mix
    wo = torch.ones(S) if w_out is None else w_out
    x.copy_(torch.einsum("tsw,sj->tjw", x, m) + wo[None, :, None] * y[:, None])
    return x


def _seq_ranges(T, slots, cu_q):
    n = len(slots)
    if cu_q is None:
        return [(s, s, s + 1) for s in range(n)]
    return [(s, int(cu_q[s]), int(cu_q[s + 1])) for s in range(n)]


def short_conv(x, w, bias, state, state_off, slots, cu_q, ctx_lens, heads, hd,
               act_silu, rot_dims, positions, inv_freq):
    """Causal per-channel convolution of x [T, C] (C = heads*hd) with w
    [C, taps]; earlier inputs of a sequence come from state[slot, i,
    state_off:state_off+C] (the input of position ctx - (taps-1) + i), zeros
    before position 0. Optional bias, SiLU, and an interleaved rotary turn of
    the first rot_dims channels of every head. Returns [T, C] in x's dtype."""
    T, C = x.shape
    taps = w.shape[1]
    K1 = taps - 1
    out = torch.zeros(T, C, dtype=torch.float32)
    wf = w.float()
    for s, t0, t1 in _seq_ranges(T, slots, cu_q):
        ctx, slot = int(ctx_lens[s]), int(slots[s])
        hist = torch.zeros(K1, C, dtype=torch.float32)
        if slot >= 0 and K1:
            hist = state[slot, :, state_off:state_off + C].float().clone()
        for i in range(K1):                 # positions before the sequence
            if ctx - K1 + i < 0:
                hist[i] = 0.0
        u = torch.cat([hist, x[t0:t1].float()], 0)
        for j in range(taps):
            out[t0:t1] += wf[:, j] * u[j:j + (t1 - t0)]
    if bias is not None:
        out += bias.float()
    if act_silu:
        out = torch.nn.functional.silu(out)
    if rot_dims:
        out = rope_interleaved(out.view(T, heads, hd), positions, inv_freq,
                               1.0, rot_dims).reshape(T, C)
    return out.to(x.dtype)


def short_conv_state(state, x, slots, cu_q):
    """Move every sequence's convolution state past this step's rows."""
    K1 = state.shape[1]
    if K1 == 0:
        return
    for s, t0, t1 in _seq_ranges(x.shape[0], slots, cu_q):
        slot = int(slots[s])
        if slot < 0:
            continue
        u = torch.cat([state[slot], x[t0:t1].to(state.dtype)], 0)
        state[slot] = u[-K1:]


def gated_recurrence(kind, q, k, v, g, p0, p1, p2, c0, c1, state, slots, cu_q,
                     ctx_lens, groups):
    """S_t = diag(a_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t (+ skip v_t);
    kind 0 (selective state space): dt = softplus(g + p0), a = exp(-exp(p1)
    dt) per head, k = dt * k, skip = p2; q/k shared by the heads of a group.
    kind 1 (gated linear attention): a = sigmoid(g + p0)^c0 per key channel,
    q scaled by c1. state fp32 [slots, H, D, Dv]; returns fp32 [T, H, Dv]."""
    H, D, Dv = state.shape[1:]
    T = q.shape[0]
    per = H // groups
    qf = q.float().view(T, groups, D).repeat_interleave(per, 1)
    kf = k.float().view(T, groups, D).repeat_interleave(per, 1)
    vf = v.float().view(T, H, Dv)
    if kind == 0:
        dt = torch.nn.functional.softplus(g.float() + p0, threshold=30.0)
        a = torch.exp(-torch.exp(p1) * dt)[:, :, None].expand(T, H, D)
        kf = kf * dt[:, :, None]
    else:
        z = g.float() + p0
        a = torch.exp(-torch.nn.functional.softplus(-z, threshold=30.0) * c0) \
            .view(T, H, D)
        qf = qf * c1
    out = torch.zeros(T, H, Dv, dtype=torch.float32)
    for s, t0, t1 in _seq_ranges(T, slots, cu_q):
        slot = int(slots[s])
        if slot >= 0 and int(ctx_lens[s]) > 0:
            S = state[slot].clone()
        else:
            S = torch.zeros(H, D, Dv, dtype=torch.float32)
        for t in range(t0, t1):
            S = a[t][:, :, None] * S + kf[t][:, :, None] * vf[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        if slot >= 0:
            state[slot] = S
    if kind == 0 and p2 is not None:
        out = out + p2[None, :, None] * vf
    return out


def gated_group_norm(o, w, gate, eps, groups, act_silu, gate_first,
                     out_dtype):
    """RMS norm over `groups` equal parts of fp32 o [rows, n], times w (n
    or n/groups entries, repeating), with gate silu/sigmoid applied before
    or after the norm."""
    act = torch.nn.functional.silu if act_silu else torch.sigmoid
    a = act(gate.float())
    z = o.float() * a if gate_first else o.float()
    rows, n = z.shape
    zg = z.view(rows, groups, n // groups)
    zg = zg * torch.rsqrt(zg.pow(2).mean(-1, keepdim=True) + eps)
    wf = w.float()
    if wf.numel() != n:
        wf = wf.repeat(groups)
    z = zg.reshape(rows, n) * wf
    if not gate_first:
        z = z * a
    return z.to(out_dtype)


def store_paged(x, cache, slot_mapping):
    """x [T, heads*hd] into cache [blocks, heads, block, hd] at the slots."""
    nb, heads, bs, hd = cache.shape
    ok = slot_mapping >= 0
    sl = slot_mapping[ok]
    cache[sl // bs, :, sl % bs] = x[ok].view(-1, heads, hd).to(cache.dtype)


def capped_attn(q, k_cache, v_cache, block_tables, cu_q, seq_lens, heads,
                scale, cap, window=0, sink=None, keep_first=0,
                head_scale=None):
    """Causal softmax attention of q [T, heads*D] over the paged caches
    [blocks, n_kv, block, D|Dv]; scores scale * q.k, then cap * tanh(. /
    cap) when cap > 0. window > 0: position i sees only the keys j with
    i - j < window. sink [heads]: exp(sink_h) joins the softmax denominator
    (a key without a value). keep_first: with a window, the keys j <
    keep_first stay visible as well. head_scale [heads]: one more score
    multiplier per head. Returns fp32 [T, heads, Dv]."""
    T = q.shape[0]
    nb, n_kv, bs, D = k_cache.shape
    Dv = v_cache.shape[3]
    per = heads // n_kv
    out = torch.zeros(T, heads, Dv, dtype=torch.float32)
    if cu_q is None:
        cu_q = torch.arange(T + 1, dtype=torch.int32)
    for s in range(len(seq_lens)):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        L = int(seq_lens[s])
        ctx = L - (q1 - q0)
        nblk = (L + bs - 1) // bs
        idx = block_tables[s][:nblk].long()
        kk = k_cache[idx].float().permute(1, 0, 2, 3).reshape(n_kv, -1, D)[:, :L]
        vv = v_cache[idx].float().permute(1, 0, 2, 3).reshape(n_kv, -1, Dv)[:, :L]
        kk = kk.repeat_interleave(per, 0)
        vv = vv.repeat_interleave(per, 0)
        qq = q[q0:q1].float().view(q1 - q0, heads, D)
        sc = torch.einsum("thd,hld->thl", qq, kk) * scale
        if head_scale is not None:
            sc = sc * head_scale.float()[None, :, None]
        if cap and cap > 0:
            sc = cap * torch.tanh(sc / cap)
        qpos = (ctx + torch.arange(q1 - q0))[:, None]
        mask = torch.arange(L)[None, :] > qpos
        if window and window > 0:
            gone = torch.arange(L)[None, :] <= qpos - window
            if keep_first > 0:
                gone = gone & (torch.arange(L)[None, :] >= keep_first)
            mask = mask | gone
        sc = sc.masked_fill(mask[:, None, :], float("-inf"))
        if sink is None:
            p = torch.softmax(sc, -1)
        else:
            sk = sink.float()[None, :, None]
            m = torch.maximum(sc.max(-1, keepdim=True).values, sk)
            e = torch.exp(sc - m)
            p = e / (e.sum(-1, keepdim=True) + torch.exp(sk - m))
        out[q0:q1] = torch.einsum("thl,hlv->thv", p, vv)
    return out


# ---------------------------------------------------------------------------
# Post-norm residual, whole-row query/key norm with rotate-half positions,
# gated delta rule, GELU-gated feed-forward. fp32 throughout.
# ---------------------------------------------------------------------------
def norm_residual_add(x, y, w1, eps, out_dtype, w_next=None):
    """x (fp32, in place) += y / rms(y) * w1; returns x in out_dtype, or
    with w_next the next sublayer's input x / rms(x) * w_next."""
    yf = y.float()
    x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * w1)
    if w_next is None:
        return x.to(out_dtype)
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
            * w_next).to(out_dtype)


def rope_halves(x, positions, inv_freq, rot_dims):
    """Entry i < rot_dims/2 of the last dim of x [T, H, D] turns together
    with entry i + rot_dims/2 by pos * inv_freq[i] (fp64 angles)."""
    if not rot_dims:
        return x.float()
    half = rot_dims // 2
    a = positions.double()[:, None] * inv_freq.double()[None, :]
    cos, sin = torch.cos(a).float()[:, None, :], torch.sin(a).float()[:, None, :]
    xf = x.float()
    u, v = xf[..., :half], xf[..., half:rot_dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin,
                      xf[..., rot_dims:]], -1)


def rownorm_rope_store(q, k, v, q_w, k_w, eps, positions, inv_freq, rot_dims,
                       heads, kv_heads, k_cache, v_cache, slot_mapping):
    """q [T, heads*D] and k [T, kv_heads*D]: RMS norm over the whole row
    times q_w / k_w, then the rotate-half turn per head. Returns the new
    q; k and v [T, kv_heads*Dv] go to the paged caches."""
    T = q.shape[0]

    def norm(z, w):
        zf = z.float()
        return zf * torch.rsqrt(zf.pow(2).mean(-1, keepdim=True) + eps) * w
    qn = rope_halves(norm(q, q_w).view(T, heads, -1), positions, inv_freq,
                     rot_dims)
    kn = rope_halves(norm(k, k_w).view(T, kv_heads, -1), positions, inv_freq,
                     rot_dims)
    store_paged(kn.reshape(T, -1).to(k.dtype), k_cache, slot_mapping)
    store_paged(v, v_cache, slot_mapping)
    return qn.reshape(T, -1).to(q.dtype)


def delta_rule(q, k, v, b, a, dt_bias, A_log, state, slots, cu_q, ctx_lens,
               groups):
    """Gated delta rule. Per head, with unit k and q (q also times
    D^-1/2), beta = sigmoid(b), g = exp(-exp(A_log) softplus(a + dt_bias)):
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q. q/k
    [T, groups*D] shared by the heads of a group; state fp32
    [slots, H, D, Dv]; returns fp32 [T, H, Dv]."""
    H, D, Dv = state.shape[1:]
    T = q.shape[0]
    per = H // groups

    def unit(z):
        zf = z.float().view(T, groups, D)
        zf = zf * torch.rsqrt(zf.pow(2).sum(-1, keepdim=True) + 1e-6)
        return zf.repeat_interleave(per, 1)
    qf, kf = unit(q) * D ** -0.5, unit(k)
    vf = v.float().view(T, H, Dv)
    beta = torch.sigmoid(b.float())
    g = torch.exp(-torch.exp(A_log) * torch.nn.functional.softplus(
        a.float() + dt_bias, threshold=30.0))
    out = torch.zeros(T, H, Dv, dtype=torch.float32)
    for s, t0, t1 in _seq_ranges(T, slots, cu_q):
        slot = int(slots[s])
        if slot >= 0 and int(ctx_lens[s]) > 0:
            S = state[slot].clone()
        else:
            S = torch.zeros(H, D, Dv, dtype=torch.float32)
        for t in range(t0, t1):
            S = g[t][:, None, None] * S
            u = beta[t][:, None] * (vf[t] - torch.einsum("hdv,hd->hv", S,
                                                         kf[t]))
            S = S + kf[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        if slot >= 0:
            state[slot] = S
    return out


def gelu_tanh_mul(x):
    """[..., 2F] -> gelu_tanh(x[..., :F]) * x[..., F:], dtype preserved."""
    return gelu_and_mul(x)


# ---------------------------------------------------------------------------
# Rotary turn + unit norm per head with paged store, PolyNorm, GELU gate of
# two tensors. fp32 throughout.
# ---------------------------------------------------------------------------
def rope_headnorm_store(q, k, v, positions, inv_freq, rot_dims, pairs,
                        unit_norm, eps, heads, kv_heads, k_cache, v_cache,
                        slot_mapping):
    """q [T, heads*D], k [T, kv_heads*D]: rotary turn on the first rot_dims
    entries of every head (`pairs`: entries 2i and 2i+1 turn together, else
    i and i + rot_dims/2), then with `unit_norm` every head is divided by
    its root mean square. Returns the new q; k and v (when given) go to the
    paged caches."""
    T = q.shape[0]

    def prep(z, n):
        z = z.reshape(T, n, -1)
        if rot_dims:
            z = (rope_interleaved(z.float(), positions, inv_freq, 1.0,
                                  rot_dims) if pairs
                 else rope_halves(z, positions, inv_freq, rot_dims))
        z = z.float()
        if unit_norm:
            z = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps)
        return z.reshape(T, -1)
    store_paged(prep(k, kv_heads).to(k.dtype), k_cache, slot_mapping)
    if v is not None:
        store_paged(v, v_cache, slot_mapping)
    return prep(q, heads).to(q.dtype)


def polynorm(z, coef, eps):
    """c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with N(u) = u / rms(u) over the
    last axis; coef fp32 [4]. dtype preserved."""
    zf = z.float()

    def unit(u):
        return u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    out = (coef[0] * unit(zf) + coef[1] * unit(zf * zf)
           + coef[2] * unit(zf * zf * zf) + coef[3])
    return out.to(z.dtype)


def gelu_tanh_gate(g, u):
    """gelu_tanh(g) * u for two tensors of one shape, dtype of g."""
    return (F.gelu(g.float(), approximate="tanh") * u.float()).to(g.dtype)
