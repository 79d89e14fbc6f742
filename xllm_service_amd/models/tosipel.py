"""Tosipel: a hybrid decoder on the paged-cache / state-slot engine.

Each layer has one sequence mixer — softmax attention over a sliding window
with a per-head sink, latent attention without positions, or a gated delta
rule recurrence — and an optional dense feed-forward gated by tanh-GELU.
The sublayers read the residual x as it is; only their OUTPUT is normed:

    x <- x + rms(mixer(x)) * (1 + w1)
    x <- x + rms(ff(x))    * (1 + w2)

The residual is fp32; what a sublayer multiplies is x rounded to the model
dtype, written by the same kernel that adds to the residual. A layer may use
another layer's weights (`weights_of`); it still owns its cache and state, so
caches are laid out per layer while the weight blocks are kept once.

fp32: residual, norms, rotary angles, scores and softmax, sink, decays, the
delta recurrence and its state. Model dtype: GEMMs, convolutions, gates.
Everything a mixer reads from its input comes out of ONE merged projection
per layer.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.engine.metadata import AttnMetadata
from xllm_service_amd.models.config import TosipelConfig
from xllm_service_amd.models.mixers import (GatedDeltaRule, LatentAttention,
                                            SinkWindowAttention)
from xllm_service_amd.ops import hybrid as hops


def _f32(n, fill=1.0):
    return nn.Parameter(torch.full((n,), fill, dtype=torch.float32))


class TosipelBlock(nn.Module):
    """The weights of one layer; run once per layer that uses them."""

    def __init__(self, cfg: TosipelConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        W, eps = cfg.hidden_size, cfg.rms_eps
        self.eps, self.dtype = eps, dtype
        m = lc.mixer
        if lc.type == "attention":
            self.mixer = SinkWindowAttention(
                W, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                m.get("rot"), m["scale"], (m.get("mask") or {}).get("size", 0),
                eps, dtype)
        elif lc.type == "latent_attention":
            self.mixer = LatentAttention(
                W, m["heads"], m["dim"], 0, m["vdim"], m["kv_rank"],
                m["scale"], None, eps, None, dtype, q_rank=m["q_rank"],
                gated=False)
        else:
            self.mixer = GatedDeltaRule(
                W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"],
                eps, dtype)
        self.in_proj = nn.Parameter(torch.empty(self.mixer.in_width, W,
                                                dtype=dtype))
        # norm weights hold 1 + w of the checkpoint
        self.norm1 = _f32(W)
        self.ff = lc.mlp is not None
        if self.ff:
            ff = lc.mlp["ff"]
            self.gate_up = nn.Parameter(torch.empty(2 * ff, W, dtype=dtype))
            self.down = nn.Parameter(torch.empty(W, ff, dtype=dtype))
            self.norm2 = _f32(W)

    def forward(self, x, h, positions, cache, meta, aux):
        """x: fp32 residual (updated in place); h: x in the model dtype.
        Returns the new x in the model dtype."""
        y = self.mixer(F.linear(h, self.in_proj), positions, cache, meta, aux)
        h = hops.norm_residual_add_(x, y, self.norm1, self.eps, self.dtype)
        if self.ff:
            y = F.linear(hops.gelu_tanh_mul(F.linear(h, self.gate_up)),
                         self.down)
            h = hops.norm_residual_add_(x, y, self.norm2, self.eps,
                                        self.dtype)
        return h


class TosipelForCausalLM(nn.Module):
    def __init__(self, cfg: TosipelConfig, dtype=torch.bfloat16):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W = cfg.hidden_size
        self.embed = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        owners = cfg.weight_layers
        self.own = sorted(set(owners))          # layers holding tensors
        self.blocks = nn.ModuleList(
            [TosipelBlock(cfg, i, dtype) for i in self.own])
        # block index of every layer, in execution order
        self.block_of: List[int] = [self.own.index(j) for j in owners]
        self.final_norm = _f32(W)
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                                dtype=dtype))

    def cache_specs(self):
        """One entry per layer: layers that share weights own their caches."""
        return [self.blocks[b].mixer.cache_spec() for b in self.block_of]

    # ---- weights -----------------------------------------------------------
    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, final.norm, head, and per layer with
        tensors of its own l<i>.{norm1,norm2}, l<i>.mlp.{gate,up,down} and
        l<i>.mix.* (attention: q, k, v, q.norm, k.norm, sink, g, o; latent
        attention: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, o; delta: q, k, v
        (each with .conv), b, a, A_log, dt_bias, norm, g, o). Norm weights
        norm1/norm2/final.norm are stored around zero (applied as 1 + w)."""
        used = set()

        def take(name):
            if name not in tensors:
                raise KeyError(f"checkpoint lacks {name!r}")
            used.add(name)
            return tensors[name]

        def put(param, value):
            if tuple(param.shape) != tuple(value.shape):
                raise ValueError(f"shape mismatch: {tuple(value.shape)} "
                                 f"for {tuple(param.shape)}")
            with torch.no_grad():
                param.copy_(value.to(param.dtype))

        def put_one_plus(param, value):
            put(param, 1.0 + value.float())

        put(self.embed.weight, take("embed"))
        put_one_plus(self.final_norm, take("final.norm"))
        put(self.lm_head, take("head"))
        for i, blk in zip(self.own, self.blocks):
            p = f"l{i}."
            m, mx = p + "mix.", blk.mixer
            if isinstance(mx, SinkWindowAttention):
                put(blk.in_proj, torch.cat([take(m + n) for n in "qkvg"], 0))
                put(mx.q_norm, take(m + "q.norm"))
                put(mx.k_norm, take(m + "k.norm"))
                put(mx.sink, take(m + "sink"))
            elif isinstance(mx, LatentAttention):
                put(blk.in_proj, torch.cat([take(m + "dq"),
                                            take(m + "dkv")], 0))
                put(mx.dq_norm, take(m + "dq.norm"))
                put(mx.dkv_norm, take(m + "dkv.norm"))
                put(mx.w_uq, take(m + "uq"))
                H, r = mx.heads, mx.kv_rank
                put(mx.w_uk, take(m + "uk").view(H, mx.dim, r))
                put(mx.w_uv_t,
                    take(m + "uv").view(H, mx.vdim, r).transpose(1, 2))
            else:
                put(blk.in_proj, torch.cat(
                    [take(m + n) for n in ("q", "k", "v", "g", "b", "a")], 0))
                put(mx.conv_w, torch.cat(
                    [take(f"{m}{n}.conv") for n in "qkv"], 0))
                put(mx.A_log, take(m + "A_log"))
                put(mx.dt_bias, take(m + "dt_bias"))
                put(mx.out_norm, take(m + "norm"))
            put(mx.o_proj, take(m + "o"))
            put_one_plus(blk.norm1, take(p + "norm1"))
            if blk.ff:
                put(blk.gate_up, torch.cat([take(p + "mlp.gate"),
                                            take(p + "mlp.up")], 0))
                put(blk.down, take(p + "mlp.down"))
                put_one_plus(blk.norm2, take(p + "norm2"))
        extra = set(tensors) - used
        if extra:
            raise ValueError(f"unused checkpoint tensors: {sorted(extra)[:8]}")

    def random_init(self, seed: int = 0):
        dev = next(self.parameters()).device
        gen = torch.Generator(device=dev).manual_seed(seed)

        def randn(shape):
            return torch.randn(shape, generator=gen, device=dev,
                               dtype=torch.float32)
        with torch.no_grad():
            for name, p in self.named_parameters():
                leaf = name.rsplit(".", 1)[-1]
                if leaf in ("dt_bias", "sink"):
                    p.copy_(0.5 * randn(p.shape))
                elif leaf == "A_log":
                    p.copy_(-1.0 + 0.5 * randn(p.shape))
                elif leaf == "conv_w":
                    p.copy_((randn(p.shape) * 0.5).to(p.dtype))
                elif leaf == "weight" and name.startswith("embed"):
                    p.copy_((randn(p.shape) / self.cfg.embed_scale)
                            .to(p.dtype))
                elif p.dtype == torch.float32 and p.dim() == 1:
                    p.copy_(1.0 + 0.1 * randn(p.shape))
                else:
                    std = 1.0 / math.sqrt(p.shape[-1])
                    p.copy_((randn(p.shape) * std).to(p.dtype))

    # ---- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches: List,
                meta: AttnMetadata,
                inputs_embeds: Optional[torch.Tensor] = None):
        e = inputs_embeds if inputs_embeds is not None \
            else self.embed(input_ids)
        x = e.float() * self.cfg.embed_scale
        h = x.to(self.dtype)
        aux = {}
        if meta.num_decode_tokens:
            aux["decode_ctx_lens"] = meta.decode_seq_lens - 1
        for i, b in enumerate(self.block_of):
            h = self.blocks[b](x, h, positions, kv_caches[i], meta, aux)
        return hops.group_rmsnorm(x, self.final_norm, self.cfg.rms_eps, 1,
                                  self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head)
