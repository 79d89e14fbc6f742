"""Model configuration + named presets (random-init; no network access)."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class ModelConfig:
    name: str = "llama"
    architecture: str = "llama"   # llama | opt | qwen2 | qwen2_vl | pugovik | dunusun | tosipel | gararax
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    max_position: int = 8192
    rms_eps: float = 1e-5
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    # vision tower (qwen2_vl only)
    vision: dict = field(default_factory=dict)
    image_pad_token_id: int = -1
    # M-RoPE frequency split (temporal, height, width) in frequency units,
    # summing to rot_dim // 2. Empty = plain 1-D RoPE.
    # (reference: Qwen2-VL 3-D rotary position embedding)
    mrope_section: tuple = ()

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim


PRESETS = {
    # flagship bench model
    "llama-3-8b": ModelConfig(
        name="llama-3-8b", vocab_size=128256, hidden_size=4096,
        intermediate_size=14336, num_layers=32, num_heads=32, num_kv_heads=8,
        head_dim=128, rope_theta=500000.0, max_position=8192),
    # small CPU-path / test configs
    "llama-tiny": ModelConfig(
        name="llama-tiny", vocab_size=1024, hidden_size=256,
        intermediate_size=512, num_layers=2, num_heads=4, num_kv_heads=2,
        head_dim=64, rope_theta=10000.0, max_position=2048),
    "llama-debug-128": ModelConfig(
        name="llama-debug-128", vocab_size=512, hidden_size=512,
        intermediate_size=1024, num_layers=2, num_heads=4, num_kv_heads=2,
        head_dim=128, rope_theta=10000.0, max_position=2048),
    # OPT-125m (CPU control-plane check)
    "opt-125m": ModelConfig(
        name="opt-125m", architecture="opt", vocab_size=50272,
        hidden_size=768, intermediate_size=3072, num_layers=12, num_heads=12,
        num_kv_heads=12, head_dim=64, max_position=2048, hidden_act="gelu"),
    # Qwen2-7B (text-only: the VL language tower without a vision stage)
    "qwen2-7b": ModelConfig(
        name="qwen2-7b", architecture="qwen2", vocab_size=152064,
        hidden_size=3584, intermediate_size=18944, num_layers=28,
        num_heads=28, num_kv_heads=4, head_dim=128, rope_theta=1000000.0,
        max_position=8192),
    "qwen2-tiny": ModelConfig(
        name="qwen2-tiny", architecture="qwen2", vocab_size=1024,
        hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4,
        num_kv_heads=2, head_dim=64, rope_theta=10000.0, max_position=2048),
    # Qwen2-VL-7B — language tower dims
    "qwen2-vl-7b": ModelConfig(
        name="qwen2-vl-7b", architecture="qwen2_vl", vocab_size=152064,
        hidden_size=3584, intermediate_size=18944, num_layers=28,
        num_heads=28, num_kv_heads=4, head_dim=128, rope_theta=1000000.0,
        max_position=8192, image_pad_token_id=151655,
        mrope_section=(16, 24, 24),
        vision=dict(depth=32, embed_dim=1280, num_heads=16, patch_size=14,
                    spatial_merge_size=2, out_hidden_size=3584)),
    # small multimodal config with head_dim 128 for GPU tests
    "qwen2-vl-debug": ModelConfig(
        name="qwen2-vl-debug", architecture="qwen2_vl", vocab_size=1024,
        hidden_size=512, intermediate_size=1024, num_layers=2, num_heads=4,
        num_kv_heads=2, head_dim=128, rope_theta=10000.0, max_position=2048,
        image_pad_token_id=9, mrope_section=(16, 24, 24),
        vision=dict(depth=2, embed_dim=256, num_heads=4, patch_size=14,
                    spatial_merge_size=2, out_hidden_size=512)),
    # tiny multimodal config with the MFMA head_dim (GPU EPD checks)
    "qwen2-vl-tiny128": ModelConfig(
        name="qwen2-vl-tiny128", architecture="qwen2_vl", vocab_size=1024,
        hidden_size=512, intermediate_size=1024, num_layers=2, num_heads=4,
        num_kv_heads=2, head_dim=128, rope_theta=10000.0, max_position=2048,
        image_pad_token_id=9, mrope_section=(16, 24, 24),
        vision=dict(depth=2, embed_dim=64, num_heads=4, patch_size=14,
                    spatial_merge_size=2, out_hidden_size=512)),
    # tiny multimodal config for CPU EPD tests
    "qwen2-vl-tiny": ModelConfig(
        name="qwen2-vl-tiny", architecture="qwen2_vl", vocab_size=1024,
        hidden_size=256, intermediate_size=512, num_layers=2, num_heads=4,
        num_kv_heads=2, head_dim=64, rope_theta=10000.0, max_position=2048,
        image_pad_token_id=9, mrope_section=(8, 12, 12),
        vision=dict(depth=2, embed_dim=64, num_heads=4, patch_size=14,
                    spatial_merge_size=2, out_hidden_size=256)),
}


@dataclass
class HybridLayerConfig:
    """One layer of a hybrid stack: which sequence mixer it has, the
    mixer's sizes and constants, and its feed-forward (None = no FF)."""
    type: str                      # latent_attention | lightning | ...
    mixer: dict = field(default_factory=dict)
    mlp: Optional[dict] = None
    # index of the layer whose tensors this layer uses (None: its own)
    weights_of: Optional[int] = None


@dataclass
class PugovikConfig(ModelConfig):
    """Pugovik: per-layer choice of latent attention (a low-rank shared
    key/value latent, optionally borrowed from an earlier layer) or decayed
    linear attention with a recurrent state, routed-expert feed-forwards,
    grouped RMS norms around every sublayer, gated + scaled residuals."""
    layers: List[HybridLayerConfig] = field(default_factory=list)
    norm_groups: int = 1
    residual_mult: float = 1.0
    model_dir: Optional[str] = None     # weights live here (None = random)

    @property
    def has_recurrent_state(self) -> bool:
        return any(l.type == "lightning" for l in self.layers)


def pugovik_from_dict(d: dict, name: str = "pugovik",
                      model_dir: Optional[str] = None) -> PugovikConfig:
    layers = [HybridLayerConfig(type=l["type"], mixer=dict(l["mixer"]),
                                mlp=l.get("mlp"))
              for l in d["layers"]]
    for i, l in enumerate(layers):
        if l.type not in ("latent_attention", "lightning"):
            raise ValueError(f"layer {i}: unknown mixer type {l.type!r}")
        src = l.mixer.get("kv_from")
        if src is not None:
            s = layers[src]
            if (src >= i or s.type != "latent_attention"
                    or "kv_from" in s.mixer):
                raise ValueError(f"layer {i}: kv_from {src} is not an earlier "
                                 "latent-attention layer with its own latent")
    return PugovikConfig(
        name=name, architecture="pugovik", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), num_layers=len(layers),
        rms_eps=float(d["norm"]["eps"]),
        norm_groups=int(d["norm"].get("groups", 1)),
        residual_mult=float(d.get("residual_mult", 1.0)),
        max_position=1 << 20, layers=layers, model_dir=model_dir)


@dataclass
class DunusunConfig(ModelConfig):
    """Dunusun: layers of a selective state space mixer (`mamba2`) or of a
    soft-capped softmax attention beside a gated linear attention
    (`parallel`), dense squared-ReLU feed-forwards, layer norms with bias,
    several residual streams mixed around every sublayer, a run of layers
    that repeats with the same weights, soft-capped logits."""
    layers: List[HybridLayerConfig] = field(default_factory=list)
    streams: Optional[int] = None       # None: one plain residual
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    logit_softcap: Optional[float] = None
    model_dir: Optional[str] = None     # weights live here (None = random)

    @property
    def layer_runs(self) -> List[int]:
        """Layer index of every layer run, in execution order (a looped
        layer appears once per pass; each run owns its cache and state)."""
        n = len(self.layers)
        body = list(range(self.loop_start, self.loop_stop))
        return (list(range(self.loop_start)) + body * self.loop_times
                + list(range(self.loop_stop, n)))

    @property
    def has_recurrent_state(self) -> bool:
        return True


def dunusun_from_dict(d: dict, name: str = "dunusun",
                      model_dir: Optional[str] = None) -> DunusunConfig:
    layers = [HybridLayerConfig(type=l["type"], mixer=dict(l["mixer"]),
                                mlp=l.get("mlp"))
              for l in d["layers"]]
    for i, l in enumerate(layers):
        if l.type not in ("mamba2", "parallel"):
            raise ValueError(f"layer {i}: unknown mixer type {l.type!r}")
        if l.mlp is not None and l.mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind")
    lp = d.get("loop") or {}
    start, stop = int(lp.get("start", 0)), int(lp.get("stop", 0))
    times = int(lp.get("times", 1))
    if not lp:
        start = stop = 0
        times = 1
    if not (0 <= start <= stop <= len(layers)) or times < 0:
        raise ValueError("loop: need 0 <= start <= stop <= layers")
    streams = d.get("streams")
    cap = d.get("logit_softcap")
    return DunusunConfig(
        name=name, architecture="dunusun", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), num_layers=len(layers),
        rms_eps=float(d["norm"]["eps"]), max_position=1 << 20, layers=layers,
        streams=None if streams is None else int(streams),
        loop_start=start, loop_stop=stop, loop_times=times,
        logit_softcap=float(cap) if cap else None, model_dir=model_dir)


@dataclass
class TosipelConfig(ModelConfig):
    """Tosipel: layers of windowed softmax attention with a sink (`attention`),
    latent attention without positions (`latent_attention`) or a gated delta
    rule recurrence (`delta`); the sublayers read the residual as it is and
    only their output is RMS-normed; dense GELU-gated feed-forwards; a layer
    may use another layer's weights with a cache of its own."""
    layers: List[HybridLayerConfig] = field(default_factory=list)
    embed_scale: float = 1.0
    model_dir: Optional[str] = None     # weights live here (None = random)

    @property
    def weight_layers(self) -> List[int]:
        """For every layer the index of the layer that owns its tensors."""
        return [i if l.weights_of is None else l.weights_of
                for i, l in enumerate(self.layers)]

    @property
    def has_recurrent_state(self) -> bool:
        return any(l.type == "delta" for l in self.layers)


def tosipel_from_dict(d: dict, name: str = "tosipel",
                      model_dir: Optional[str] = None) -> TosipelConfig:
    layers = [HybridLayerConfig(type=l["type"], mixer=dict(l["mixer"]),
                                mlp=l.get("mlp"),
                                weights_of=l.get("weights_of"))
              for l in d["layers"]]
    for i, l in enumerate(layers):
        if l.type not in ("attention", "latent_attention", "delta"):
            raise ValueError(f"layer {i}: unknown mixer type {l.type!r}")
        if l.mlp is not None and l.mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind")
    for i, l in enumerate(layers):
        seen = {i}
        while l.weights_of is not None:       # follow a chain to its owner
            j = int(l.weights_of)
            if not 0 <= j < len(layers) or j in seen:
                raise ValueError(f"layer {i}: bad weights_of {j}")
            seen.add(j)
            owner = layers[j]
            if owner.type != layers[i].type:
                raise ValueError(f"layer {i}: weights_of {j} is another "
                                 "kind of layer")
            if owner.weights_of is None:
                layers[i].weights_of = j
                break
            l = owner
    return TosipelConfig(
        name=name, architecture="tosipel", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), num_layers=len(layers),
        rms_eps=float(d["norm"]["eps"]),
        embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
        max_position=1 << 20, layers=layers, model_dir=model_dir)


@dataclass
class GararaxConfig(ModelConfig):
    """Gararax: layers of grouped-head softmax attention in three kinds
    (`attention`: pair-layout rotary with banded frequency scaling, unit RMS
    norm of q and k, sliding window that also keeps the first tokens;
    `attention_2`: no positions, values are the keys, a sink of score 0,
    sigmoid output gate; `attention_3`: biased projections, half-layout
    rotary, one score multiplier per head, every earlier key), RMS norms
    before and after every sublayer, a scaled residual, dense PolyNorm or
    routed-expert feed-forwards, a small per-layer token embedding added
    after the feed-forward, a run of layers that repeats with the same
    weights, and the embedding table as the head."""
    layers: List[HybridLayerConfig] = field(default_factory=list)
    residual_mult: float = 1.0
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    side_dim: int = 0                   # per-layer token embedding (0: none)
    model_dir: Optional[str] = None     # weights live here (None = random)

    @property
    def layer_runs(self) -> List[int]:
        """Layer index of every layer run, in execution order (a looped
        layer appears once per pass; each run owns its cache)."""
        n = len(self.layers)
        body = list(range(self.loop_start, self.loop_stop))
        return (list(range(self.loop_start)) + body * self.loop_times
                + list(range(self.loop_stop, n)))

    @property
    def has_recurrent_state(self) -> bool:
        return False


GARARAX_MIXERS = ("attention", "attention_2", "attention_3")


def gararax_from_dict(d: dict, name: str = "gararax",
                      model_dir: Optional[str] = None) -> GararaxConfig:
    layers = [HybridLayerConfig(type=l["type"], mixer=dict(l["mixer"]),
                                mlp=l.get("mlp"))
              for l in d["layers"]]
    for i, l in enumerate(layers):
        if l.type not in GARARAX_MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {l.type!r}")
        if l.mlp is not None and l.mlp.get("kind") not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind")
        if l.type == "attention_2" and \
                l.mixer.get("vdim", l.mixer["dim"]) != l.mixer["dim"]:
            raise ValueError(f"layer {i}: values are keys, vdim must be dim")
    lp = d.get("loop") or {}
    start, stop = int(lp.get("start", 0)), int(lp.get("stop", 0))
    times = int(lp.get("times", 1))
    if not lp or stop <= start:
        start = stop = 0
        times = 1
    if not (0 <= start <= stop <= len(layers)) or times < 1:
        raise ValueError("loop: need 0 <= start <= stop <= layers, times >= 1")
    return GararaxConfig(
        name=name, architecture="gararax", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), num_layers=len(layers),
        rms_eps=float(d["norm"]["eps"]),
        residual_mult=float(d.get("residual_mult", 1.0)),
        loop_start=start, loop_stop=stop, loop_times=times,
        side_dim=int((d.get("token_side") or {}).get("dim", 0)),
        max_position=1 << 20, layers=layers, model_dir=model_dir)


def load_model_dir(path: str) -> ModelConfig:
    """Read <path>/config.json and pick the config class by its
    `architecture` field."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = str(d.get("architecture", "")).lower()
    if arch == "pugovik":
        return pugovik_from_dict(d, name=os.path.basename(
            os.path.normpath(path)) or "pugovik", model_dir=path)
    if arch == "dunusun":
        return dunusun_from_dict(d, name=os.path.basename(
            os.path.normpath(path)) or "dunusun", model_dir=path)
    if arch == "tosipel":
        return tosipel_from_dict(d, name=os.path.basename(
            os.path.normpath(path)) or "tosipel", model_dir=path)
    if arch == "gararax":
        return gararax_from_dict(d, name=os.path.basename(
            os.path.normpath(path)) or "gararax", model_dir=path)
    raise ValueError(f"{path}: unsupported architecture "
                     f"{d.get('architecture')!r}")


def _pugovik_preset(name, width, n_layers, heads, vocab=32000, experts=16,
                    top=2, ff=None, every_attn=4, kv_rank=512, rot_dim=64):
    """Synthetic Pugovik stacks for benchmarks: three decayed-linear layers
    per latent-attention layer, the second attention layer of each pair
    borrowing the first one's latent."""
    hd = width // heads
    layers, last_attn = [], None
    for i in range(n_layers):
        mlp = dict(kind="moe", expert=dict(ff=ff or width // 2),
                   router=dict(experts=experts, top=top,
                               groups=dict(count=4, keep=2)))
        if i % every_attn == every_attn - 1:
            mixer = dict(heads=heads, dim=hd, rot_dim=rot_dim, vdim=hd,
                         kv_rank=kv_rank, scale=(hd + rot_dim) ** -0.5,
                         rot=dict(base=10000.0, dims=rot_dim))
            if last_attn is not None:
                mixer["kv_from"] = last_attn
                last_attn = None
            else:
                last_attn = i
            layers.append(dict(type="latent_attention", mixer=mixer, mlp=mlp))
        else:
            decay = [1.0 - 2.0 ** -(2 + 6 * h / max(heads - 1, 1))
                     for h in range(heads)]
            layers.append(dict(type="lightning", mlp=mlp, mixer=dict(
                heads=heads, dim=hd, vdim=hd, decay=decay)))
    return pugovik_from_dict(dict(
        architecture="Pugovik", vocab=vocab, width=width, layers=layers,
        norm=dict(eps=1e-6, groups=4), residual_mult=0.5), name=name)


def _llama_equal(name, width, n_layers, heads, vocab=32000, ff=None):
    """Llama stack of the same width, depth and active feed-forward size
    as the pugovik bench stack of that width (comparison baseline)."""
    return ModelConfig(name=name, vocab_size=vocab, hidden_size=width,
                       intermediate_size=ff or width, num_layers=n_layers,
                       num_heads=heads, num_kv_heads=max(heads // 4, 1),
                       head_dim=width // heads, rope_theta=10000.0,
                       max_position=16384)


PRESETS.update({
    "llama-2k": _llama_equal("llama-2k", 2048, 8, 16),
    "llama-4k": _llama_equal("llama-4k", 4096, 8, 32),
    # CPU-test sized hybrid stack
    "pugovik-tiny": _pugovik_preset("pugovik-tiny", 128, 4, 4, vocab=256,
                                    experts=8, top=2, ff=64, every_attn=2,
                                    kv_rank=48, rot_dim=16),
    # bench stacks at the width of real deployments (random weights)
    "pugovik-2k": _pugovik_preset("pugovik-2k", 2048, 8, 16),
    "pugovik-4k": _pugovik_preset("pugovik-4k", 4096, 8, 32),
})


def _dunusun_preset(name, width, n_layers, vocab=32000, every_attn=4,
                    streams=2, head=128, state=128, loop=None):
    """Synthetic Dunusun stacks for benchmarks: three selective state space
    layers per parallel (attention + gated linear attention) layer, a dense
    feed-forward of 1.5 x width in every layer."""
    layers = []
    mlp = dict(kind="dense", ff=3 * width // 2)
    for i in range(n_layers):
        if i % every_attn == every_attn - 1:
            heads = max(width // head, 1)
            left = dict(heads=heads, kv_heads=max(heads // 4, 1), dim=head,
                        vdim=head, conv=4, scale=head ** -0.5, softcap=50.0,
                        rot=dict(base=10000.0, dims=head // 2))
            right = dict(heads=max(heads // 4, 1), dim=head, vdim=head,
                         tau=16.0, rank=32)
            layers.append(dict(type="parallel", mlp=mlp, mixer=dict(
                left=left, right=right, left_scale=1.0, right_scale=1.0)))
        else:
            sh = max(width // (head // 2), 1)
            layers.append(dict(type="mamba2", mlp=mlp, mixer=dict(
                heads=sh, vdim=head // 2, state=state,
                groups=max(sh // 4, 1), norm_groups=max(sh // 4, 1), conv=4)))
    d = dict(architecture="Dunusun", vocab=vocab, width=width, layers=layers,
             norm=dict(eps=1e-6), streams=streams, logit_softcap=30.0)
    if loop:
        d["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return dunusun_from_dict(d, name=name)


PRESETS.update({
    # CPU-test sized stack (the second layer runs twice)
    "dunusun-tiny": _dunusun_preset("dunusun-tiny", 64, 3, vocab=256,
                                    every_attn=2, head=16, state=8,
                                    loop=(1, 2, 2)),
    # bench stacks at the width of real deployments (random weights)
    "dunusun-2k": _dunusun_preset("dunusun-2k", 2048, 8),
    "dunusun-4k": _dunusun_preset("dunusun-4k", 4096, 8),
})


def _tosipel_preset(name, width, n_layers, vocab=32000, head=128, window=1024,
                    kv_rank=512, q_rank=None, share=True):
    """Synthetic Tosipel stacks for benchmarks: two delta-rule layers, one
    windowed attention layer and one latent attention layer per group of
    four; the second attention layer reuses the first one's weights."""
    heads = max(width // head, 1)
    ff = dict(kind="dense", ff=3 * width // 2)
    layers, first_attn = [], None
    for i in range(n_layers):
        k = i % 4
        if k == 1:
            lc = dict(type="attention", mlp=ff, mixer=dict(
                heads=heads, kv_heads=max(heads // 4, 1), dim=head, vdim=head,
                mask=dict(size=window), rot=dict(base=10000.0, dims=head // 2),
                scale=head ** -0.5))
            if first_attn is None:
                first_attn = i
            elif share:
                lc["weights_of"] = first_attn
            layers.append(lc)
        elif k == 3:
            layers.append(dict(type="latent_attention", mlp=ff, mixer=dict(
                heads=heads, dim=head, vdim=head, kv_rank=kv_rank,
                q_rank=q_rank or max(width // 2, 16), scale=head ** -0.5)))
        else:
            layers.append(dict(type="delta", mlp=ff, mixer=dict(
                heads=heads, kv_heads=max(heads // 2, 1), dim=head, vdim=head,
                conv=4)))
    return tosipel_from_dict(dict(
        architecture="Tosipel", vocab=vocab, width=width, layers=layers,
        norm=dict(eps=1e-6), embedding=dict(scale=float(width) ** 0.5)),
        name=name)


PRESETS.update({
    # CPU-test sized stack (the second attention layer shares weights)
    "tosipel-tiny": _tosipel_preset("tosipel-tiny", 64, 6, vocab=256, head=16,
                                    window=24, kv_rank=24, q_rank=20),
    # bench stacks at the width of real deployments (random weights)
    "tosipel-2k": _tosipel_preset("tosipel-2k", 2048, 8),
    "tosipel-4k": _tosipel_preset("tosipel-4k", 4096, 8),
})


def _gararax_preset(name, width, n_layers, vocab=32000, head=128, window=1024,
                    keep_first=4, experts=16, top=2, identity=2, side=64,
                    loop=None):
    """Synthetic Gararax stacks for benchmarks: per group of four layers a
    gated keys-as-values attention layer with a dense feed-forward, two
    full-context biased layers and one windowed layer with routed experts
    (plus identity experts and a shared expert)."""
    heads = max(width // head, 1)
    kv = max(heads // 4, 1)
    n_all = experts + identity
    groups = 4 if n_all % 4 == 0 and n_all >= 8 else 1
    moe = dict(kind="moe", expert=dict(ff=width // 2),
               router=dict(experts=experts, top=top, identity=identity,
                           groups=dict(count=groups,
                                       keep=max(groups // 2, 1))),
               shared=dict(ff=width // 2))
    dense = dict(kind="dense", ff=3 * width // 2)
    layers = []
    for i in range(n_layers):
        k = i % 4
        if k == 0:
            layers.append(dict(type="attention_2", mlp=dense, mixer=dict(
                heads=heads, kv_heads=kv, dim=head, vdim=head,
                mask=dict(size=window, keep_first=keep_first),
                scale=head ** -0.5)))
        elif k == 3:
            layers.append(dict(type="attention", mlp=moe, mixer=dict(
                heads=heads, kv_heads=kv, dim=head, vdim=head,
                mask=dict(size=window, keep_first=keep_first),
                rot=dict(base=10000.0, dims=head // 2, scaling=dict(
                    factor=8.0, low=1.0, high=4.0, original=8192)),
                scale=1.0)))
        else:
            layers.append(dict(type="attention_3", mlp=moe, mixer=dict(
                heads=heads, kv_heads=kv, dim=head, vdim=head,
                rot=dict(base=10000.0, dims=head), scale=head ** -0.5)))
    d = dict(architecture="Gararax", vocab=vocab, width=width, layers=layers,
             norm=dict(eps=1e-6), residual_mult=0.5)
    if side:
        d["token_side"] = dict(dim=side)
    if loop:
        d["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return gararax_from_dict(d, name=name)


PRESETS.update({
    # CPU-test sized stack (layers 1..2 run twice)
    "gararax-tiny": _gararax_preset("gararax-tiny", 64, 4, vocab=256, head=16,
                                    window=20, keep_first=3, experts=6, top=2,
                                    identity=2, side=8, loop=(1, 3, 2)),
    # bench stacks at the width of real deployments (random weights)
    "gararax-2k": _gararax_preset("gararax-2k", 2048, 8),
    "gararax-4k": _gararax_preset("gararax-4k", 4096, 8),
})


def get_config(name: str) -> ModelConfig:
    if os.path.isdir(name):
        return load_model_dir(name)
    if name not in PRESETS:
        raise KeyError(f"unknown model preset {name!r}; have {list(PRESETS)}")
    return PRESETS[name]
