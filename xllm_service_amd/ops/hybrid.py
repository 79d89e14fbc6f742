"""Hybrid-mixer ops: latent attention, decayed linear attention with a
recurrent state, grouped RMS norms, gated residuals, routed experts;
residual streams, short convolutions, gated recurrences, soft-capped and
windowed paged attention; post-norm residual, whole-row q/k norm with
rotate-half positions, the gated delta rule.

Same policy as the rest of `ops`: on a GPU the HIP extension (`_ops_hybrid`)
is the only path and its absence raises; on CPU the fp32 torch references in
`ops.ref` run. Activations may be bf16 or fp32; norms, scores, softmax
weights, recurrent state, router and residual are fp32 in both.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ref

_ext = None


def _hyb():
    global _ext
    if _ext is None:
        try:
            from xllm_service_amd import _ops_hybrid as m
        except ImportError as e:
            raise RuntimeError(
                "xllm_service_amd._ops_hybrid (gfx950 HIP extension) is not "
                "built but a GPU op was requested. Build it with: "
                "XLLM_BUILD_EXT=_ops_hybrid python setup.py build_ext "
                "--inplace") from e
        _ext = m
    return _ext


def group_rmsnorm(x, w, eps: float, groups: int, out_dtype=None):
    out_dtype = out_dtype or x.dtype
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _hyb().group_rmsnorm(out, x, w, eps, groups)
        return out
    return ref.group_rmsnorm(x, w, eps, groups, out_dtype)


def gated_norm_residual(res, y, gate, gate_bias, w, ls, mult: float,
                        eps: float, groups: int):
    """res (fp32, in place) += mult * ls * group_rmsnorm(y * sigmoid(gate +
    gate_bias)) * w."""
    if res.is_cuda:
        _hyb().gated_norm_residual(res, y, gate, gate_bias, w, ls, mult, eps,
                                   groups)
        return res
    return ref.gated_norm_residual(res, y, gate, gate_bias, w, ls, mult, eps,
                                   groups)


def norm_sigmoid_gate(o, w: Optional[torch.Tensor], gate, eps: float,
                      out_dtype, gate_cols: int = 1):
    """(rmsnorm(o) * w if w is given else o) * sigmoid(gate); o fp32 2-D.
    gate_cols > 1: gate has o's width / gate_cols entries per row, each
    serving that many neighbouring columns (one gate per head)."""
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        _hyb().norm_sigmoid_gate(out, o, w, gate, eps, gate_cols)
        return out
    return ref.norm_sigmoid_gate(o, w, gate, eps, out_dtype, gate_cols)


def silu_mul(x):
    if x.is_cuda:
        out = torch.empty(x.shape[:-1] + (x.shape[-1] // 2,), dtype=x.dtype,
                          device=x.device)
        _hyb().silu_mul(out, x)
        return out
    return ref.silu_mul(x)


def rope_interleaved_(x, positions, inv_freq, mscale: float, off: int,
                      rot_dims: int):
    """Rotate x[..., off:off+rot_dims] ([T, H, D] view) in place."""
    if x.is_cuda:
        _hyb().rope_interleaved(x, positions, inv_freq, mscale, off, rot_dims)
        return x
    x[..., off:off + rot_dims] = ref.rope_interleaved(
        x[..., off:off + rot_dims], positions, inv_freq, mscale, rot_dims)
    return x


def latent_kv_store(dkv, norm_w, eps, positions, inv_freq, mscale, rot_dims,
                    cache, slot_mapping, kv_rank):
    if dkv.is_cuda:
        _hyb().latent_kv_store(cache, dkv, norm_w, eps, positions, inv_freq,
                               mscale, rot_dims, slot_mapping, kv_rank)
        return
    ref.latent_kv_store(dkv, norm_w, eps, positions, inv_freq, mscale,
                        rot_dims, cache, slot_mapping, kv_rank)


def latent_attn(q, cache, block_tables, cu_q, seq_lens, scale, kv_rank, out):
    """out fp32 [T, H, kv_rank] (written). cu_q None: decode rows."""
    if q.is_cuda:
        _hyb().latent_attn(out, q, cache, block_tables, cu_q, seq_lens, scale,
                           kv_rank)
        return out
    if cu_q is None:
        cu_q = torch.arange(q.shape[0] + 1, dtype=torch.int32)
    out.copy_(ref.latent_attn(q, cache, block_tables, cu_q, seq_lens, scale,
                              kv_rank))
    return out


def decay_attn(q, k, v, decay, state, slots, cu_q, ctx_lens, out,
               max_q_len: int = 0):
    """out fp32 [T, H, Dv] (written); q/k/v are pre-activation row views
    [T, H*D] / [T, H*Dv]; state fp32 [slots, H, D, Dv] updated in place.
    max_q_len: host-known bound on the longest sequence chunk (0: unknown)."""
    if q.is_cuda:
        _hyb().decay_attn(out, q, k, v, decay, state, slots, cu_q, ctx_lens,
                          max_q_len)
        return out
    H, D, Dv = state.shape[1:]
    T = q.shape[0]
    if cu_q is None:
        cu_q = torch.arange(T + 1, dtype=torch.int32)
    out.copy_(ref.decay_linear_attn(
        q.reshape(T, H, D), k.reshape(T, H, D), v.reshape(T, H, Dv), decay,
        state, slots, cu_q, ctx_lens))
    return out


def moe_route(h, w_router, top: int, n_groups: int, keep: int, *,
              softmax: bool = False, correction=None, group_max: bool = False,
              normalize: bool = False):
    """Router: fp32 logits h @ w_router^T (a true-fp32 library GEMM on the
    GPU; h enters as stored, i.e. possibly bf16-rounded), then the scores
    (sigmoid, or softmax over all experts) and the group-limited top-k
    selection kernel. correction fp32 [experts] is added to the scores for
    the choice only; group_max scores a group by its best expert instead of
    its two best; normalize divides the chosen weights by their sum."""
    if h.is_cuda:
        T = h.shape[0]
        z = torch.matmul(h.float(), w_router.t())
        ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
        wts = torch.empty(T, top, dtype=torch.float32, device=h.device)
        _hyb().moe_route(ids, wts, z, top, n_groups, keep, softmax,
                         correction, group_max, normalize)
        return ids, wts
    return ref.moe_route(h, w_router, top, n_groups, keep, softmax,
                         correction, group_max, normalize)


def moe_combine(y, rows, wts, tokens: int, ident=None, extra=None):
    """fp32 [tokens, width] = sum_k wts[t, k] * y[rows[t, k]] (+ extra[t]).
    A negative row stands for the token's own input: ident[t]."""
    width = y.shape[-1]
    if y.is_cuda:
        out = torch.empty(tokens, width, dtype=torch.float32, device=y.device)
        _hyb().moe_combine(out, y.view(-1, width), rows, wts, ident, extra)
        return out
    yy = y.reshape(-1, width).float()[rows.long().clamp(min=0)]   # [T,top,W]
    if ident is not None:
        yy = torch.where((rows < 0)[:, :, None], ident.float()[:, None, :], yy)
    out = (yy * wts[:, :, None]).sum(1)
    return out if extra is None else out + extra.float()


# ---- residual streams, short convolutions, gated recurrences ---------------
def streams_mix_norm(x, w_in: Optional[torch.Tensor], g, b, eps: float,
                     out_dtype):
    """Layer norm (weight g, bias b) of sum_s w_in[s] x[:, s]; x fp32
    [T, S, W] -> [T, W]."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], x.shape[2], dtype=out_dtype,
                          device=x.device)
        _hyb().streams_mix_norm(out, x, w_in, g, b, eps)
        return out
    return ref.streams_mix_norm(x, w_in, g, b, eps, out_dtype)


def streams_update_(x, mix, w_out, y1, a1: float = 1.0, y2=None,
                    a2: float = 0.0):
    """x[:, j] <- sum_s mix[s, j] x[:, s] + w_out[j] (a1 y1 + a2 y2), in
    place on the fp32 streams [T, S, W]; mix / w_out None = identity / 1."""
    if x.is_cuda:
        _hyb().streams_update(x, mix, w_out, y1, a1, y2, a2)
        return x
    return ref.streams_update(x, mix, w_out, y1, a1, y2, a2)


def streams_update_mix_norm_(x, mix, w_out, y1, a1, y2, a2, w_in, g, b,
                             eps: float):
    """streams_update_ followed by streams_mix_norm of the new values (the
    next sublayer's read) in one pass; returns the normed input in y1's
    dtype."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], x.shape[2], dtype=y1.dtype,
                          device=x.device)
        _hyb().streams_update_mix_norm(out, x, mix, w_out, y1, a1, y2, a2,
                                       w_in, g, b, eps)
        return out
    ref.streams_update(x, mix, w_out, y1, a1, y2, a2)
    return ref.streams_mix_norm(x, w_in, g, b, eps, y1.dtype)


def relu_sq_(x):
    if x.is_cuda:
        _hyb().relu_sq(x)
        return x
    return x.copy_(torch.relu(x.float()).pow(2).to(x.dtype))


def softcap(x, cap: float):
    """fp32 cap * tanh(x / cap)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        _hyb().softcap(out, x.contiguous(), cap)
        return out
    return cap * torch.tanh(x.float() / cap)


def short_conv(x, w, bias, state, state_off: int, slots, cu_q, ctx_lens,
               heads: int, hd: int, *, act_silu: bool = False,
               rot_dims: int = 0, positions=None, inv_freq=None,
               cache=None, slot_mapping=None):
    """Short causal convolution with carried inputs (see ref.short_conv).
    With `cache` [blocks, heads, block, hd] the result is scattered to the
    tokens' slots and None is returned; else a new [T, heads*hd] tensor."""
    if x.is_cuda:
        out = None
        if cache is None:
            out = torch.empty(x.shape[0], heads * hd, dtype=x.dtype,
                              device=x.device)
        _hyb().short_conv(out, cache, slot_mapping, x, w, bias, state,
                          state_off, slots, cu_q, ctx_lens, heads, hd,
                          act_silu, rot_dims, positions, inv_freq)
        return out
    out = ref.short_conv(x, w, bias, state, state_off, slots, cu_q, ctx_lens,
                         heads, hd, act_silu, rot_dims, positions, inv_freq)
    if cache is None:
        return out
    ref.store_paged(out, cache, slot_mapping)
    return None


def short_conv_state_(state, x, slots, cu_q):
    """After every reader of the old state ran: keep the last taps-1 rows."""
    if state.shape[1] == 0:
        return
    if x.is_cuda:
        _hyb().short_conv_state(state, x, slots, cu_q)
        return
    ref.short_conv_state(state, x, slots, cu_q)


def gated_recurrence(kind: int, q, k, v, g, p0, p1, p2, c0: float, c1: float,
                     state, slots, cu_q, ctx_lens, groups: int, out,
                     max_q_len: int = 0):
    """out fp32 [T, H, Dv] (written); see ref.gated_recurrence."""
    if q.is_cuda:
        _hyb().gated_recurrence(kind, out, q, k, v, g, p0, p1, p2, c0, c1,
                                state, slots, cu_q, ctx_lens, groups,
                                max_q_len)
        return out
    out.copy_(ref.gated_recurrence(kind, q, k, v, g, p0, p1, p2, c0, c1,
                                   state, slots, cu_q, ctx_lens, groups))
    return out


def gated_group_norm(o, w, gate, eps: float, groups: int, *, act_silu: bool,
                     gate_first: bool, out_dtype):
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        _hyb().gated_group_norm(out, o, w, gate, eps, groups, act_silu,
                                gate_first)
        return out
    return ref.gated_group_norm(o, w, gate, eps, groups, act_silu,
                                gate_first, out_dtype)


def capped_attn(q, k_cache, v_cache, block_tables, cu_q, seq_lens,
                heads: int, scale: float, cap: float, out, window: int = 0,
                sink: Optional[torch.Tensor] = None, keep_first: int = 0,
                head_scale: Optional[torch.Tensor] = None):
    """out fp32 [T, heads, Dv] (written). cu_q None: decode rows. window > 0
    limits a query to the last `window` keys (itself included) and, with
    keep_first, the first keep_first keys of the sequence; sink fp32 [heads]
    adds exp(sink_h) to the softmax denominator; head_scale fp32 [heads]
    multiplies the scores of a head."""
    if window <= 0:
        keep_first = 0
    if q.is_cuda:
        _hyb().capped_attn(out, q, k_cache, v_cache, block_tables, cu_q,
                           seq_lens, heads, scale, cap, window, sink,
                           keep_first, head_scale)
        return out
    out.copy_(ref.capped_attn(q, k_cache, v_cache, block_tables, cu_q,
                              seq_lens, heads, scale, cap, window, sink,
                              keep_first, head_scale))
    return out


# ---- post-norm residual, whole-row q/k norm, delta rule, GELU gate ----------
def norm_residual_add_(x, y, w1, eps: float, out_dtype, w_next=None):
    """x (fp32 [T, W], in place) += y / rms(y) * w1 (y fp32 or model dtype).
    Returns the new x in out_dtype, or with w_next the following sublayer's
    normed input x / rms(x) * w_next from the same pass."""
    if x.is_cuda:
        h = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _hyb().norm_residual_add(x, h, y, w1, eps, w_next)
        return h
    return ref.norm_residual_add(x, y, w1, eps, out_dtype, w_next)


def rownorm_rope_store(q, k, v, q_w, k_w, eps: float, positions, inv_freq,
                       rot_dims: int, heads: int, kv_heads: int, k_cache,
                       v_cache, slot_mapping):
    """RMS norm of the whole q row [T, heads*D] and k row [T, kv_heads*D]
    (weights q_w, k_w), rotate-half positions on the first rot_dims entries
    of every head. Returns the new q as a contiguous tensor; k and v go
    into the paged caches at the tokens' slots."""
    if q.is_cuda:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        _hyb().rownorm_rope_store(out, q, k, v, q_w, k_w, eps, positions,
                                  inv_freq, rot_dims, heads, kv_heads,
                                  k_cache, v_cache, slot_mapping)
        return out
    return ref.rownorm_rope_store(q, k, v, q_w, k_w, eps, positions,
                                  inv_freq, rot_dims, heads, kv_heads,
                                  k_cache, v_cache, slot_mapping)


def delta_rule(q, k, v, b, a, dt_bias, A_log, state, slots, cu_q, ctx_lens,
               groups: int, out, max_q_len: int = 0):
    """out fp32 [T, H, Dv] (written); see ref.delta_rule. q/k/v/b/a are row
    views of the projections; state fp32 [slots, H, D, Dv] in place.
    max_q_len: host-known bound on the longest sequence chunk (0: unknown)."""
    if q.is_cuda:
        _hyb().delta_rule(out, q, k, v, b, a, dt_bias, A_log, state, slots,
                          cu_q, ctx_lens, groups, max_q_len)
        return out
    out.copy_(ref.delta_rule(q, k, v, b, a, dt_bias, A_log, state, slots,
                             cu_q, ctx_lens, groups))
    return out


def gelu_tanh_mul(x):
    """[..., 2F] -> gelu_tanh(x[..., :F]) * x[..., F:]."""
    if x.is_cuda:
        out = torch.empty(x.shape[:-1] + (x.shape[-1] // 2,), dtype=x.dtype,
                          device=x.device)
        _hyb().gelu_tanh_mul(out, x)
        return out
    return ref.gelu_tanh_mul(x)


# ---- rotary + unit head norm with paged store, PolyNorm, two-tensor gate ----
def rope_headnorm_store(q, k, v, positions, inv_freq, rot_dims: int,
                        pairs: bool, unit_norm: bool, eps: float, heads: int,
                        kv_heads: int, k_cache, v_cache, slot_mapping):
    """Rotary turn on the first rot_dims entries of every head of q [T,
    heads*D] and k [T, kv_heads*D] (`pairs`: entries 2i / 2i+1, else i / i +
    rot_dims/2), then with unit_norm each head divided by its root mean
    square. Returns the new q as a contiguous tensor; k and v (None: the
    values are the keys) go into the paged caches at the tokens' slots."""
    if q.is_cuda:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        _hyb().rope_headnorm_store(out, q, k, v, positions, inv_freq,
                                   rot_dims, pairs, unit_norm, eps, heads,
                                   kv_heads, k_cache, v_cache, slot_mapping)
        return out
    return ref.rope_headnorm_store(q, k, v, positions, inv_freq, rot_dims,
                                   pairs, unit_norm, eps, heads, kv_heads,
                                   k_cache, v_cache, slot_mapping)


def polynorm(z, coef, eps: float):
    """coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3] per row, N =
    division by the root mean square of the row; fp32 inside."""
    if z.is_cuda:
        out = torch.empty(z.shape, dtype=z.dtype, device=z.device)
        _hyb().polynorm(out, z, coef, eps)
        return out
    return ref.polynorm(z, coef, eps)


def gelu_tanh_gate(g, u):
    """gelu_tanh(g) * u, g and u [T, F] row views of one dtype."""
    if g.is_cuda:
        out = torch.empty(g.shape, dtype=g.dtype, device=g.device)
        _hyb().gelu_tanh_gate(out, g, u)
        return out
    return ref.gelu_tanh_gate(g, u)
