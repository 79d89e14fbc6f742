"""Gararax: an attention decoder on the paged-cache engine.

Each layer has one grouped-head attention mixer of three kinds and an
optional feed-forward, each between two RMS norms, and then a small
per-layer token embedding is gated into the residual:

    x <- x + m * norm1b(mixer(norm1(x)))
    x <- x + m * norm2b(ff(norm2(x)))
    g  = gelu_tanh(W_gate x) * side_embed[token][layer part]
    x <- x + m * rms(W_proj g) * w_side

`attention`   rotary in the pair layout with banded frequency scaling, unit
              RMS norm of q and k per head, sliding window + kept first keys
`attention_2` no positions, the keys are the values, a sink of score 0 in
              the softmax, element-wise sigmoid output gate
`attention_3` biased projections, rotary in the half layout, one score
              multiplier per head, every earlier key

Feed-forwards: dense with PolyNorm (a weighted sum of the unit-normed first
three powers), or routed experts (softmax router, a correction for the
choice, groups scored by their best member, identity experts, a shared
expert). A run of consecutive layers may repeat with the same weights; every
pass owns its caches, so caches are laid out per layer RUN. Before every
pass a learned step vector is added to the residual, and from the second
pass on the token embedding as well. The head is the embedding table.

fp32: residual, norms (PolyNorm included), rotary angles, scores and
softmax, router. Model dtype: GEMMs, gates, activations. Everything a mixer
reads from its input comes out of ONE merged projection per layer. The
residual multiplier m is folded into the weights of the norms that write
into the residual; each such write also forms the next sublayer's normed
input in the same pass over the row.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.engine.metadata import AttnMetadata
from xllm_service_amd.models.config import GararaxConfig
from xllm_service_amd.models.mixers import GroupedAttention
from xllm_service_amd.models.moe import RoutedExperts
from xllm_service_amd.ops import hybrid as hops


def _f32(*shape, fill=1.0):
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32))


def make_mixer(kind: str, m: dict, width: int, eps: float, dtype):
    mask = m.get("mask") or {}
    common = dict(width=width, heads=m["heads"], kv_heads=m["kv_heads"],
                  dim=m["dim"], vdim=m.get("vdim", m["dim"]),
                  scale=m["scale"], window=mask.get("size", 0),
                  keep_first=mask.get("keep_first", 0), norm_eps=eps,
                  dtype=dtype)
    if kind == "attention":
        return GroupedAttention(rot=m.get("rot"), rot_pairs=True,
                                unit_norm=True, **common)
    if kind == "attention_2":
        return GroupedAttention(rot=None, rot_pairs=True, zero_sink=True,
                                values_are_keys=True, gated=True, **common)
    if kind == "attention_3":
        return GroupedAttention(rot=m.get("rot"), rot_pairs=False,
                                head_scale=True, **common)
    raise ValueError(f"unknown mixer type {kind!r}")


class PolyNormFF(nn.Module):
    """down(polynorm(up h))."""

    def __init__(self, width: int, ff: int, eps: float, dtype):
        super().__init__()
        self.eps = eps
        self.up = nn.Parameter(torch.empty(ff, width, dtype=dtype))
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype))
        self.coef = _f32(4)

    def forward(self, h):
        return F.linear(hops.polynorm(F.linear(h, self.up), self.coef,
                                      self.eps), self.down)


class GararaxBlock(nn.Module):
    """The weights of one layer; run once per pass that uses them."""

    def __init__(self, cfg: GararaxConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        W, eps = cfg.hidden_size, cfg.rms_eps
        self.eps, self.dtype, self.index = eps, dtype, index
        self.mixer = make_mixer(lc.type, lc.mixer, W, eps, dtype)
        self.in_proj = nn.Parameter(torch.empty(self.mixer.in_width, W,
                                                dtype=dtype))
        self.in_bias = nn.Parameter(torch.zeros(
            self.mixer.in_width, dtype=dtype)) \
            if lc.type == "attention_3" else None
        # norm1b / norm2b / side_norm hold residual_mult * w of the checkpoint
        self.norm1, self.norm1b = _f32(W), _f32(W)
        self.ff = None
        if lc.mlp is not None:
            self.norm2, self.norm2b = _f32(W), _f32(W)
            if lc.mlp["kind"] == "dense":
                self.ff = PolyNormFF(W, lc.mlp["ff"], eps, dtype)
            else:
                r = lc.mlp["router"]
                g = r.get("groups") or {}
                self.ff = RoutedExperts(
                    W, lc.mlp["expert"]["ff"], r["experts"], r["top"],
                    g.get("count", 1), g.get("keep", 1), dtype,
                    identity=r.get("identity", 0), softmax=True,
                    correction=True, group_max=True, normalize=True,
                    shared_ff=(lc.mlp.get("shared") or {}).get("ff", 0))
        self.side = cfg.side_dim
        if self.side:
            self.side_gate = nn.Parameter(torch.empty(self.side, W,
                                                      dtype=dtype))
            self.side_proj = nn.Parameter(torch.empty(W, self.side,
                                                      dtype=dtype))
            self.side_norm = _f32(W)

    def forward(self, x, h, side_e, positions, cache, meta, aux, next_w):
        """x: fp32 residual (updated in place); h: norm1(x) in the model
        dtype. Returns what follows the layer: the residual normed with
        next_w, or the residual itself in the model dtype (next_w None)."""
        eps, dt = self.eps, self.dtype
        y = self.mixer(F.linear(h, self.in_proj, self.in_bias), positions,
                       cache, meta, aux)
        last = None if self.side else next_w
        h = hops.norm_residual_add_(
            x, y, self.norm1b, eps, dt,
            self.norm2 if self.ff is not None else last)
        if self.ff is not None:
            h = hops.norm_residual_add_(x, self.ff(h), self.norm2b, eps, dt,
                                        last)
        if self.side:
            lo = self.index * self.side
            g = hops.gelu_tanh_gate(F.linear(h, self.side_gate),
                                    side_e[:, lo:lo + self.side])
            h = hops.norm_residual_add_(x, F.linear(g, self.side_proj),
                                        self.side_norm, eps, dt, next_w)
        return h


class GararaxForCausalLM(nn.Module):
    def __init__(self, cfg: GararaxConfig, dtype=torch.bfloat16):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W, n = cfg.hidden_size, cfg.num_layers
        self.embed = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        self.side_embed = nn.Embedding(cfg.vocab_size, n * cfg.side_dim,
                                       dtype=dtype) if cfg.side_dim else None
        self.blocks = nn.ModuleList(
            [GararaxBlock(cfg, i, dtype) for i in range(n)])
        self.looped = cfg.loop_stop > cfg.loop_start
        self.loop_step = _f32(cfg.loop_times, W, fill=0.0) \
            if self.looped else None
        self.final_norm = _f32(W)
        # layer of every run, and the pass a run opens (None: it opens none)
        self.runs: List[int] = cfg.layer_runs
        body = cfg.loop_stop - cfg.loop_start
        self.opens: List[Optional[int]] = [
            (r - cfg.loop_start) // body
            if self.looped and cfg.loop_start <= r < cfg.loop_start
            + body * cfg.loop_times and (r - cfg.loop_start) % body == 0
            else None for r in range(len(self.runs))]

    def cache_specs(self):
        """One entry per layer run: every pass of a looped layer owns its
        cache."""
        return [self.blocks[i].mixer.cache_spec() for i in self.runs]

    # ---- weights -----------------------------------------------------------
    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, final.norm, side.embed, loop.step, and
        per layer l<i>.{norm1,norm1b,norm2,norm2b}, l<i>.mix.{q,k,v,g,o}
        (attention_3: q.b, k.b, v.b, temp), l<i>.mlp.{up,down,act} or
        l<i>.mlp.{router,correction,e<j>.{gate,up,down},shared.{gate,up,
        down}}, l<i>.side.{gate,proj,norm}. Linear weights are [out, in]."""
        used = set()
        mult = self.cfg.residual_mult

        def take(name):
            if name not in tensors:
                raise KeyError(f"checkpoint lacks {name!r}")
            used.add(name)
            return tensors[name]

        def put(param, value, times=None):
            if tuple(param.shape) != tuple(value.shape):
                raise ValueError(f"shape mismatch: {tuple(value.shape)} "
                                 f"for {tuple(param.shape)}")
            with torch.no_grad():
                if times is not None:
                    value = value.float() * times
                param.copy_(value.to(param.dtype))

        put(self.embed.weight, take("embed"))
        put(self.final_norm, take("final.norm"))
        if self.side_embed is not None:
            put(self.side_embed.weight, take("side.embed"))
        if self.looped:
            put(self.loop_step, take("loop.step"))
        else:
            used.add("loop.step")          # a loop over no layers adds nothing
        for i, blk in enumerate(self.blocks):
            p = f"l{i}."
            m, mx = p + "mix.", blk.mixer
            names = ["q", "k"] + ([] if mx.values_are_keys else ["v"]) \
                + (["g"] if mx.gated else [])
            put(blk.in_proj, torch.cat([take(m + n) for n in names], 0))
            if blk.in_bias is not None:
                put(blk.in_bias, torch.cat([take(m + n + ".b")
                                            for n in names], 0))
            if mx.head_scale is not None:
                put(mx.head_scale, take(m + "temp"))
            put(mx.o_proj, take(m + "o"))
            put(blk.norm1, take(p + "norm1"))
            put(blk.norm1b, take(p + "norm1b"), mult)
            ff = blk.ff
            if ff is not None:
                put(blk.norm2, take(p + "norm2"))
                put(blk.norm2b, take(p + "norm2b"), mult)
                f = p + "mlp."
                if isinstance(ff, PolyNormFF):
                    put(ff.up, take(f + "up"))
                    put(ff.down, take(f + "down"))
                    put(ff.coef, take(f + "act"))
                else:
                    put(ff.router, take(f + "router"))
                    if f + "correction" in tensors:
                        put(ff.correction, take(f + "correction"))
                    put(ff.w_gate_up, torch.stack([
                        torch.cat([take(f"{f}e{j}.gate"),
                                   take(f"{f}e{j}.up")], 0)
                        for j in range(ff.experts)]))
                    put(ff.w_down, torch.stack([take(f"{f}e{j}.down")
                                                for j in range(ff.experts)]))
                    if ff.shared_ff:
                        put(ff.shared_gate_up,
                            torch.cat([take(f + "shared.gate"),
                                       take(f + "shared.up")], 0))
                        put(ff.shared_down, take(f + "shared.down"))
            if blk.side:
                put(blk.side_gate, take(p + "side.gate"))
                put(blk.side_proj, take(p + "side.proj"))
                put(blk.side_norm, take(p + "side.norm"), mult)
        extra = set(tensors) - used
        if extra:
            raise ValueError(f"unused checkpoint tensors: {sorted(extra)[:8]}")

    def random_init(self, seed: int = 0):
        dev = next(self.parameters()).device
        gen = torch.Generator(device=dev).manual_seed(seed)
        mult = self.cfg.residual_mult

        def randn(shape):
            return torch.randn(shape, generator=gen, device=dev,
                               dtype=torch.float32)
        with torch.no_grad():
            for name, p in self.named_parameters():
                leaf = name.rsplit(".", 1)[-1]
                if leaf == "coef":
                    p.copy_(torch.tensor([0.6, 0.3, 0.1, 0.0], device=dev)
                            + 0.05 * randn(p.shape))
                elif leaf == "correction":
                    p.copy_(0.02 * randn(p.shape))
                elif leaf == "loop_step":
                    p.copy_(0.1 * randn(p.shape))
                elif leaf == "in_bias":
                    p.copy_((0.1 * randn(p.shape)).to(p.dtype))
                elif leaf in ("norm1b", "norm2b", "side_norm"):
                    p.copy_(mult * (1.0 + 0.1 * randn(p.shape)))
                elif p.dtype == torch.float32 and p.dim() == 1:
                    p.copy_(1.0 + 0.1 * randn(p.shape))
                elif leaf == "weight":                 # embedding tables
                    p.copy_(randn(p.shape).to(p.dtype))
                else:
                    std = 1.0 / math.sqrt(p.shape[-1])
                    p.copy_((randn(p.shape) * std).to(p.dtype))

    # ---- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches: List,
                meta: AttnMetadata,
                inputs_embeds: Optional[torch.Tensor] = None):
        e = inputs_embeds if inputs_embeds is not None \
            else self.embed(input_ids)
        e32 = e.float()
        x = e32.clone() if self.looped else e32
        side_e = self.side_embed(input_ids) \
            if self.side_embed is not None else None
        aux = {}
        if meta.num_decode_tokens:
            aux["decode_ctx_lens"] = meta.decode_seq_lens - 1
        eps, n_runs = self.cfg.rms_eps, len(self.runs)
        h = None
        for r, i in enumerate(self.runs):
            blk = self.blocks[i]
            t = self.opens[r]
            if t is not None:
                if t > 0:
                    x.add_(e32)
                x.add_(self.loop_step[t])
            if h is None:
                h = hops.group_rmsnorm(x, blk.norm1, eps, 1, self.dtype)
            if r + 1 == n_runs:
                next_w = self.final_norm
            elif self.opens[r + 1] is not None:
                next_w = None            # the residual changes before its norm
            else:
                next_w = self.blocks[self.runs[r + 1]].norm1
            h = blk(x, h, side_e, positions, kv_caches[r], meta, aux, next_w)
            if next_w is None:
                h = None
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.embed.weight)
