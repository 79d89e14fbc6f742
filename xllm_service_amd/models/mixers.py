"""Sequence mixers beyond plain multi-head attention.

LatentAttention        softmax attention whose keys and values are linear
                       images of one cached low-rank latent per token, plus
                       one rotated key part shared by all heads. Queries are
                       folded through the key up-projection so the kernel
                       works on the cached rows directly; the value
                       up-projection follows the weighted sum.
DecayLinearAttention   per-head state S <- decay * S + k v^T, o = S^T q with
                       SiLU feature maps; the state lives in a slot pool.

SelectiveStateSpace    Mamba-2 style mixer: short convolution + SiLU on
                       [x | B | C], per-head scalar decay exp(-exp(A) dt),
                       state S <- a S + dt B x^T, y = S^T C + D x, SiLU gate,
                       grouped RMS norm.
CappedAttention        softmax attention with grouped key/value heads, a
                       short convolution on q/k/v, rotary pairs on part of
                       each head, a tanh soft cap on the scores, separate
                       key and value widths, sigmoid output gate.
GatedLinearAttention   S <- diag(alpha) S + k v^T, o = S^T q with a low-rank
                       per-channel decay alpha = sigmoid(.)^(1/tau); RMS norm
                       per head, SiLU gate.
ParallelMixer          two mixers reading the same input, outputs added
                       with fixed weights.
SinkWindowAttention    softmax attention with grouped key/value heads over a
                       sliding window of keys, RMS norm over the whole query
                       and key projection, rotate-half positions on part of
                       each head, a learned per-head sink in the softmax
                       denominator, one sigmoid gate number per head.
GatedDeltaRule         S <- g S; u = beta (v - S^T k); S <- S + k u^T;
                       o = S^T q with unit q, k after a short convolution and
                       SiLU; per-head scalar decay g; RMS norm per head, SiLU
                       gate.
GroupedAttention       softmax attention with grouped key/value heads whose
                       parts are all options: rotary positions in the pair or
                       the half layout (plain or with banded frequency
                       scaling), unit RMS norm of q and k per head after the
                       turn, a sliding window that also keeps the first
                       tokens, a sink of score 0, one score multiplier per
                       head, keys read as values, element-wise sigmoid gate.

All take the slice of a merged input projection that belongs to them and
return the mixer output in the model dtype. Sizes and constants are
constructor arguments.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.engine.cache_spec import (CacheGroup, ConvState,
                                                PagedKV, PagedLatent,
                                                RecurrentState, SharedCache)
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


def banded_rope_frequencies(rot: dict):
    """Per-pair inverse frequencies (fp64) of a rotary config {base, dims,
    scaling?}. With `scaling` = {factor, low, high, original} a frequency f
    of wavelength l = 2 pi / f stays as it is for l < original / high,
    becomes f / factor for l > original / low, and in between is the blend
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor, low, high = float(sc["factor"]), float(sc["low"]), \
        float(sc["high"])
    orig = float(sc["original"])
    wl = 2.0 * math.pi / f
    s = (orig / wl - low) / (high - low)
    blend = (1.0 - s) * f / factor + s * f
    return torch.where(wl < orig / high, f,
                       torch.where(wl > orig / low, f / factor, blend))


class LatentAttention(nn.Module):
    """rot None (with rot_dim 0): no rotated key part, no positions.
    q_rank: the queries come from a normed low-rank latent of that size
    (the merged projection then holds the latent's rows instead of q).
    gated False: no sigmoid output gate."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int,
                 vdim: int, kv_rank: int, scale: float, rot: Optional[dict],
                 norm_eps: float, kv_from: Optional[int], dtype,
                 q_rank: Optional[int] = None, gated: bool = True):
        super().__init__()
        self.heads, self.dim, self.rot_dim = heads, dim, rot_dim
        self.vdim, self.kv_rank = vdim, kv_rank
        self.scale, self.eps, self.kv_from = float(scale), norm_eps, kv_from
        self.rot_dims = int(rot["dims"]) if rot else 0
        if self.rot_dims > rot_dim or self.rot_dims % 2:
            raise ValueError("rotary dims must be even and <= rot_dim")
        if rot:
            inv_freq, self.mscale = scaled_rope_frequencies(rot)
        else:
            inv_freq, self.mscale = torch.zeros(0, dtype=torch.float64), 1.0
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        self.q_rank, self.gated = q_rank, gated
        self.q_width = heads * (dim + rot_dim)
        self.q_in = q_rank if q_rank else self.q_width
        self.dkv_width = 0 if kv_from is not None else kv_rank + rot_dim
        self.g_width = heads * vdim if gated else 0
        # merged-projection rows owned by this mixer: [q | dkv | g]
        self.in_width = self.q_in + self.dkv_width + self.g_width
        if q_rank:
            self.dq_norm = nn.Parameter(torch.ones(q_rank,
                                                   dtype=torch.float32))
            self.w_uq = nn.Parameter(torch.empty(self.q_width, q_rank,
                                                 dtype=dtype))
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
        if self.q_rank:
            cq = hops.group_rmsnorm(proj[:, :self.q_in], self.dq_norm,
                                    self.eps, 1, proj.dtype)
            q = F.linear(cq, self.w_uq).unflatten(-1, (H, dim + rd))
        else:
            q = proj[:, :self.q_width].unflatten(-1, (H, dim + rd))
        if self.rot_dims:
            hops.rope_interleaved_(q, positions, self.inv_freq, self.mscale,
                                   dim, self.rot_dims)
        if self.kv_from is None:
            dkv = proj[:, self.q_in:self.q_in + self.dkv_width]
            hops.latent_kv_store(dkv, self.dkv_norm, self.eps, positions,
                                 self.inv_freq, self.mscale, self.rot_dims,
                                 cache, meta.slot_mapping, r)
        # fold the queries through the key up-projection: [H,T,dim]x[H,dim,r]
        q_abs = torch.bmm(q[..., :dim].transpose(0, 1), self.w_uk)
        if rd:
            qf = torch.empty(T, H, r + rd, dtype=proj.dtype,
                             device=proj.device)
            qf[..., :r] = q_abs.transpose(0, 1)
            qf[..., r:] = q[..., dim:]
        else:
            qf = q_abs.transpose(0, 1).contiguous()
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
        if not self.gated:
            return F.linear(o, self.o_proj)
        gate = proj[:, self.q_in + self.dkv_width:self.in_width]
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


def _halves(meta: AttnMetadata, aux):
    """The prefill and the decode part of a batch as (rows, cu_q, ctx_lens,
    state_slots, seq_lens, block_tables, max_len) tuples."""
    np_, nd = meta.num_prefill_tokens, meta.num_decode_tokens
    out = []
    if np_:
        out.append((slice(0, np_), meta.cu_q, meta.prefill_ctx_lens,
                    meta.prefill_state_slots, meta.prefill_seq_lens,
                    meta.prefill_block_tables, meta.max_prefill_len))
    if nd:
        out.append((slice(np_, np_ + nd), None, aux["decode_ctx_lens"],
                    meta.decode_state_slots, meta.decode_seq_lens,
                    meta.decode_block_tables, 1))
    return out


class SelectiveStateSpace(nn.Module):
    """in_proj rows: [z: inner | x: inner | B: G*N | C: G*N | dt: heads],
    inner = heads * vdim."""

    def __init__(self, width: int, heads: int, vdim: int, state: int,
                 groups: int, norm_groups: int, taps: int, norm_eps: float,
                 dtype):
        super().__init__()
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("heads % groups and inner % norm_groups must be 0")
        self.heads, self.vdim, self.state, self.groups = heads, vdim, state, \
            groups
        self.norm_groups, self.taps, self.eps = norm_groups, taps, norm_eps
        self.inner = heads * vdim
        self.conv_ch = self.inner + 2 * groups * state
        self.in_width = 2 * self.inner + 2 * groups * state + heads
        f32 = dict(dtype=torch.float32)
        self.conv_w = nn.Parameter(torch.empty(self.conv_ch, taps, dtype=dtype))
        self.conv_b = nn.Parameter(torch.zeros(self.conv_ch, dtype=dtype))
        self.dt_bias = nn.Parameter(torch.zeros(heads, **f32))
        self.A_log = nn.Parameter(torch.zeros(heads, **f32))
        self.D = nn.Parameter(torch.ones(heads, **f32))
        self.out_norm = nn.Parameter(torch.ones(self.inner, **f32))
        self.o_proj = nn.Parameter(torch.empty(width, self.inner, dtype=dtype))

    def cache_spec(self):
        return CacheGroup((ConvState(self.conv_ch, self.taps),
                           RecurrentState(self.heads, self.state, self.vdim)))

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        conv_state, ssm_state = cache
        T, inner, gn = proj.shape[0], self.inner, self.groups * self.state
        z = proj[:, :inner]
        xbc_in = proj[:, inner:inner + self.conv_ch]
        dt = proj[:, inner + self.conv_ch:self.in_width]
        o = torch.empty(T, self.heads, self.vdim, dtype=torch.float32,
                        device=proj.device)
        for rows, cu_q, ctx, slots, _, _, max_len in _halves(meta, aux):
            u = xbc_in[rows]
            xbc = hops.short_conv(u, self.conv_w, self.conv_b, conv_state, 0,
                                  slots, cu_q, ctx, 1, self.conv_ch,
                                  act_silu=True)
            hops.short_conv_state_(conv_state, u, slots, cu_q)
            hops.gated_recurrence(
                0, xbc[:, inner + gn:], xbc[:, inner:inner + gn],
                xbc[:, :inner], dt[rows], self.dt_bias, self.A_log, self.D,
                0.0, 1.0, ssm_state, slots, cu_q, ctx, self.groups, o[rows],
                max_q_len=max_len)
        y = hops.gated_group_norm(o.view(T, inner), self.out_norm, z, self.eps,
                                  self.norm_groups, act_silu=True,
                                  gate_first=True, out_dtype=proj.dtype)
        return F.linear(y, self.o_proj)


class CappedAttention(nn.Module):
    """in_proj rows: [q: heads*dim | k: kv_heads*dim | v: kv_heads*vdim |
    g: heads*vdim]."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, taps: int, rot: Optional[dict], scale: float,
                 softcap: Optional[float], dtype):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, \
            dim, vdim
        self.taps, self.scale = taps, float(scale)
        self.softcap = float(softcap) if softcap else 0.0
        self.rot_dims = int(rot["dims"]) if rot else 0
        if self.rot_dims > dim or self.rot_dims % 2:
            raise ValueError("rotary dims must be even and <= dim")
        if self.rot_dims:
            inv_freq, _ = scaled_rope_frequencies(
                dict(base=rot["base"], dims=rot["dims"]))
            self.register_buffer("inv_freq", inv_freq, persistent=False)
        else:
            self.inv_freq = None
        self.cq, self.ck, self.cv = heads * dim, kv_heads * dim, \
            kv_heads * vdim
        self.conv_ch = self.cq + self.ck + self.cv
        self.g_width = heads * vdim
        self.in_width = self.conv_ch + self.g_width
        # filters of q, k, v stacked in the order of the projection rows
        self.conv_w = nn.Parameter(torch.empty(self.conv_ch, taps, dtype=dtype))
        self.o_proj = nn.Parameter(torch.empty(width, self.g_width,
                                               dtype=dtype))

    def cache_spec(self):
        return CacheGroup((ConvState(self.conv_ch, self.taps),
                           PagedKV(self.kv_heads, self.dim, self.vdim)))

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        conv_state, (k_cache, v_cache) = cache
        T, cq, ck = proj.shape[0], self.cq, self.ck
        H, G = self.heads, self.kv_heads
        qkv = proj[:, :self.conv_ch]
        gate = proj[:, self.conv_ch:self.in_width]
        o = torch.empty(T, H, self.vdim, dtype=torch.float32,
                        device=proj.device)
        rot = dict(rot_dims=self.rot_dims, inv_freq=self.inv_freq)
        for rows, cu_q, ctx, slots, seq_lens, tables, _ in _halves(meta, aux):
            u, pos = qkv[rows], positions[rows]
            sm = meta.slot_mapping[rows]
            q = hops.short_conv(u[:, :cq], self.conv_w[:cq], None, conv_state,
                                0, slots, cu_q, ctx, H, self.dim,
                                positions=pos, **rot)
            hops.short_conv(u[:, cq:cq + ck], self.conv_w[cq:cq + ck], None,
                            conv_state, cq, slots, cu_q, ctx, G, self.dim,
                            positions=pos, cache=k_cache, slot_mapping=sm,
                            **rot)
            hops.short_conv(u[:, cq + ck:], self.conv_w[cq + ck:], None,
                            conv_state, cq + ck, slots, cu_q, ctx, G,
                            self.vdim, cache=v_cache, slot_mapping=sm)
            hops.short_conv_state_(conv_state, u, slots, cu_q)
            hops.capped_attn(q, k_cache, v_cache, tables, cu_q, seq_lens, H,
                             self.scale, self.softcap, o[rows])
        y = hops.norm_sigmoid_gate(o.view(T, self.g_width), None, gate, 0.0,
                                   proj.dtype)
        return F.linear(y, self.o_proj)


class GatedLinearAttention(nn.Module):
    """in_proj rows: [q: heads*dim | k: heads*dim | v: heads*vdim |
    g: heads*vdim | a1: rank]; the decay logits are a2 (a1 h) + a2_b."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int,
                 tau: float, rank: int, norm_eps: float, dtype):
        super().__init__()
        self.heads, self.dim, self.vdim = heads, dim, vdim
        self.tau, self.rank, self.eps = float(tau), rank, norm_eps
        self.qk_width, self.v_width = heads * dim, heads * vdim
        self.in_width = 2 * self.qk_width + 2 * self.v_width + rank
        self.a2 = nn.Parameter(torch.empty(self.qk_width, rank, dtype=dtype))
        self.a2_b = nn.Parameter(torch.zeros(self.qk_width,
                                             dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.ones(vdim, dtype=torch.float32))
        self.o_proj = nn.Parameter(torch.empty(width, self.v_width,
                                               dtype=dtype))

    def cache_spec(self):
        return RecurrentState(self.heads, self.dim, self.vdim)

    def forward(self, proj, positions, state, meta: AttnMetadata, aux):
        T, a, b = proj.shape[0], self.qk_width, self.v_width
        q, k = proj[:, :a], proj[:, a:2 * a]
        v = proj[:, 2 * a:2 * a + b]
        gate = proj[:, 2 * a + b:2 * a + 2 * b]
        z = F.linear(proj[:, 2 * a + 2 * b:self.in_width], self.a2)
        o = torch.empty(T, self.heads, self.vdim, dtype=torch.float32,
                        device=proj.device)
        for rows, cu_q, ctx, slots, _, _, max_len in _halves(meta, aux):
            hops.gated_recurrence(
                1, q[rows], k[rows], v[rows], z[rows], self.a2_b, None, None,
                1.0 / self.tau, self.dim ** -0.5, state, slots, cu_q, ctx,
                self.heads, o[rows], max_q_len=max_len)
        y = hops.gated_group_norm(o.view(T, b), self.out_norm, gate, self.eps,
                                  self.heads, act_silu=True, gate_first=False,
                                  out_dtype=proj.dtype)
        return F.linear(y, self.o_proj)


class ParallelMixer(nn.Module):
    """Two mixers on the same input; the caller adds their outputs with the
    weights `scales` (kept apart so the sum is taken in fp32)."""

    def __init__(self, left: nn.Module, right: nn.Module, left_scale: float,
                 right_scale: float):
        super().__init__()
        self.left, self.right = left, right
        self.scales = (float(left_scale), float(right_scale))
        self.in_width = left.in_width + right.in_width

    def cache_spec(self):
        return CacheGroup((self.left.cache_spec(), self.right.cache_spec()))

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        lw = self.left.in_width
        return (self.left(proj[:, :lw], positions, cache[0], meta, aux),
                self.right(proj[:, lw:self.in_width], positions, cache[1],
                           meta, aux))


class SinkWindowAttention(nn.Module):
    """in_proj rows: [q: heads*dim | k: kv_heads*dim | v: kv_heads*vdim |
    g: heads]. window 0 = every earlier key."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, rot: Optional[dict], scale: float, window: int,
                 norm_eps: float, dtype):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, \
            dim, vdim
        self.scale, self.window, self.eps = float(scale), int(window), norm_eps
        self.rot_dims = int(rot["dims"]) if rot else 0
        if self.rot_dims > dim or self.rot_dims % 2:
            raise ValueError("rotary dims must be even and <= dim")
        if self.rot_dims:
            inv_freq, _ = scaled_rope_frequencies(
                dict(base=rot["base"], dims=rot["dims"]))
        else:
            inv_freq = torch.zeros(0, dtype=torch.float64)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        self.cq, self.ck, self.cv = heads * dim, kv_heads * dim, \
            kv_heads * vdim
        self.in_width = self.cq + self.ck + self.cv + heads
        f32 = dict(dtype=torch.float32)
        self.q_norm = nn.Parameter(torch.ones(self.cq, **f32))
        self.k_norm = nn.Parameter(torch.ones(self.ck, **f32))
        self.sink = nn.Parameter(torch.zeros(heads, **f32))
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim,
                                               dtype=dtype))

    def cache_spec(self):
        return PagedKV(self.kv_heads, self.dim, self.vdim)

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        k_cache, v_cache = cache
        T, cq, ck, cv = proj.shape[0], self.cq, self.ck, self.cv
        H = self.heads
        q = hops.rownorm_rope_store(
            proj[:, :cq], proj[:, cq:cq + ck], proj[:, cq + ck:cq + ck + cv],
            self.q_norm, self.k_norm, self.eps, positions, self.inv_freq,
            self.rot_dims, H, self.kv_heads, k_cache, v_cache,
            meta.slot_mapping)
        gate = proj[:, cq + ck + cv:self.in_width]
        o = torch.empty(T, H, self.vdim, dtype=torch.float32,
                        device=proj.device)
        for rows, cu_q, _, _, seq_lens, tables, _ in _halves(meta, aux):
            hops.capped_attn(q[rows], k_cache, v_cache, tables, cu_q,
                             seq_lens, H, self.scale, 0.0, o[rows],
                             window=self.window, sink=self.sink)
        y = hops.norm_sigmoid_gate(o.view(T, H * self.vdim), None, gate, 0.0,
                                   proj.dtype, gate_cols=self.vdim)
        return F.linear(y, self.o_proj)


class GatedDeltaRule(nn.Module):
    """in_proj rows: [q: kv_heads*dim | k: kv_heads*dim | v: heads*vdim |
    g: heads*vdim | b: heads | a: heads]; q, k, v pass the short
    convolution (filters stacked in that order) and SiLU."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, taps: int, norm_eps: float, dtype):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, \
            dim, vdim
        self.taps, self.eps = taps, norm_eps
        self.qk_width, self.v_width = kv_heads * dim, heads * vdim
        self.conv_ch = 2 * self.qk_width + self.v_width
        self.in_width = self.conv_ch + self.v_width + 2 * heads
        f32 = dict(dtype=torch.float32)
        self.conv_w = nn.Parameter(torch.empty(self.conv_ch, taps, dtype=dtype))
        self.dt_bias = nn.Parameter(torch.zeros(heads, **f32))
        self.A_log = nn.Parameter(torch.zeros(heads, **f32))
        self.out_norm = nn.Parameter(torch.ones(vdim, **f32))
        self.o_proj = nn.Parameter(torch.empty(width, self.v_width,
                                               dtype=dtype))

    def cache_spec(self):
        return CacheGroup((ConvState(self.conv_ch, self.taps),
                           RecurrentState(self.heads, self.dim, self.vdim)))

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        conv_state, state = cache
        T, a, b, H = proj.shape[0], self.qk_width, self.v_width, self.heads
        c = self.conv_ch
        u_all = proj[:, :c]
        gate = proj[:, c:c + b]
        beta, dt = proj[:, c + b:c + b + H], proj[:, c + b + H:self.in_width]
        o = torch.empty(T, H, self.vdim, dtype=torch.float32,
                        device=proj.device)
        for rows, cu_q, ctx, slots, _, _, max_len in _halves(meta, aux):
            u = u_all[rows]
            x = hops.short_conv(u, self.conv_w, None, conv_state, 0, slots,
                                cu_q, ctx, 1, c, act_silu=True)
            hops.short_conv_state_(conv_state, u, slots, cu_q)
            hops.delta_rule(x[:, :a], x[:, a:2 * a], x[:, 2 * a:], beta[rows],
                            dt[rows], self.dt_bias, self.A_log, state, slots,
                            cu_q, ctx, self.kv_heads, o[rows],
                            max_q_len=max_len)
        y = hops.gated_group_norm(o.view(T, b), self.out_norm, gate, self.eps,
                                  H, act_silu=True, gate_first=False,
                                  out_dtype=proj.dtype)
        return F.linear(y, self.o_proj)


class GroupedAttention(nn.Module):
    """in_proj rows: [q: heads*dim | k: kv_heads*dim | v: kv_heads*vdim
    (absent with values_are_keys) | g: heads*vdim (with gated)].

    rot: {base, dims, scaling?} or None; rot_pairs: entries (2i, 2i+1) turn
    together, else (i, i + dims/2). unit_norm: q and k are divided by their
    root mean square per head after the turn. window 0 = every earlier key;
    keep_first: the first keys stay visible beside the window. zero_sink: 1
    joins the softmax denominator. head_scale: a learned score multiplier
    per head. values_are_keys: the weighted sum runs over the cached keys.
    gated: the heads' outputs are multiplied by sigmoid(g)."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, rot: Optional[dict], rot_pairs: bool,
                 scale: float, window: int, keep_first: int, norm_eps: float,
                 dtype, *, unit_norm: bool = False, zero_sink: bool = False,
                 head_scale: bool = False, values_are_keys: bool = False,
                 gated: bool = False):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if values_are_keys and vdim != dim:
            raise ValueError("keys read as values: vdim must equal dim")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, \
            dim, vdim
        self.scale, self.eps = float(scale), norm_eps
        self.window, self.keep_first = int(window), int(keep_first)
        self.rot_pairs, self.unit_norm = bool(rot_pairs), bool(unit_norm)
        self.values_are_keys, self.gated = values_are_keys, gated
        self.rot_dims = int(rot["dims"]) if rot else 0
        if self.rot_dims > dim or self.rot_dims % 2:
            raise ValueError("rotary dims must be even and <= dim")
        inv_freq = banded_rope_frequencies(rot) if self.rot_dims \
            else torch.zeros(0, dtype=torch.float64)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        self.cq, self.ck = heads * dim, kv_heads * dim
        self.cv = 0 if values_are_keys else kv_heads * vdim
        self.g_width = heads * vdim if gated else 0
        self.in_width = self.cq + self.ck + self.cv + self.g_width
        f32 = dict(dtype=torch.float32)
        if zero_sink:
            self.register_buffer("sink", torch.zeros(heads, **f32),
                                 persistent=False)
        else:
            self.sink = None
        self.head_scale = nn.Parameter(torch.ones(heads, **f32)) \
            if head_scale else None
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim,
                                               dtype=dtype))

    def cache_spec(self):
        return PagedKV(self.kv_heads, self.dim, self.vdim,
                       values_are_keys=self.values_are_keys)

    def forward(self, proj, positions, cache, meta: AttnMetadata, aux):
        k_cache, v_cache = cache
        T, cq, ck, cv = proj.shape[0], self.cq, self.ck, self.cv
        H = self.heads
        v_in = proj[:, cq + ck:cq + ck + cv] if cv else None
        q = hops.rope_headnorm_store(
            proj[:, :cq], proj[:, cq:cq + ck], v_in, positions, self.inv_freq,
            self.rot_dims, self.rot_pairs, self.unit_norm, self.eps, H,
            self.kv_heads, k_cache, v_cache, meta.slot_mapping)
        o = torch.empty(T, H, self.vdim, dtype=torch.float32,
                        device=proj.device)
        for rows, cu_q, _, _, seq_lens, tables, _ in _halves(meta, aux):
            hops.capped_attn(q[rows], k_cache, v_cache, tables, cu_q,
                             seq_lens, H, self.scale, 0.0, o[rows],
                             window=self.window, sink=self.sink,
                             keep_first=self.keep_first,
                             head_scale=self.head_scale)
        o = o.view(T, H * self.vdim)
        if self.gated:
            y = hops.norm_sigmoid_gate(
                o, None, proj[:, cq + ck + cv:self.in_width], 0.0, proj.dtype)
        else:
            y = o.to(proj.dtype)
        return F.linear(y, self.o_proj)
