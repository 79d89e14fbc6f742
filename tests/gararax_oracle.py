"""Plain, slow implementation of the Gararax decoder, one function per
mechanism, written from the equations and sharing no code with the engine.

Everything works on one whole sequence at a time (no cache, no batching):
`forward(cfg, weights, tokens)` returns the logits at every position and the
residual after every layer run. `cfg` is the parsed config.json dictionary
and `weights` maps checkpoint tensor names to tensors. All arithmetic runs
in `dtype` (float64 by default).
"""
from __future__ import annotations

import math

import torch


# ---- small pieces -----------------------------------------------------------
def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def linear(x, w, b=None):
    y = x @ w.T
    return y if b is None else y + b


# ---- rotary positions -------------------------------------------------------
def rotary_frequencies(rot, dtype=torch.float64):
    """f_i = base^(-2i/dims), optionally rescaled by wavelength bands: short
    wavelengths keep f, long ones use f / factor, a linear blend between."""
    dims = int(rot["dims"])
    i = torch.arange(dims // 2, dtype=dtype)
    f = float(rot["base"]) ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor, low, high = float(sc["factor"]), float(sc["low"]), float(sc["high"])
    orig = float(sc["original"])
    out = f.clone()
    for j in range(dims // 2):
        wl = 2.0 * math.pi / float(f[j])
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[j] = f[j] / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[j] = (1.0 - s) * f[j] / factor + s * f[j]
    return out


def rotate(x, positions, freqs, dims, layout):
    """x [T, H, D]: turn the first `dims` entries of every head by the angle
    position * f_i. layout 'pairs': entries (2i, 2i+1) form pair i; 'halves':
    entries (i, i + dims/2)."""
    if dims == 0:
        return x
    ang = positions.to(x.dtype)[:, None] * freqs.to(x.dtype)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if layout == "pairs":
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


# ---- attention --------------------------------------------------------------
def visible(T, window, keep_first):
    """mask[i, j]: position i sees j. window None = every earlier key."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if window is not None:
        m = m & ((i - j < window) | (j < keep_first))
    return m


def attend(q, k, v, scale, mask, head_scale=None, sink=False):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; softmax over the visible keys
    (with `sink`, 1 joins the denominator)."""
    T, H, _ = q.shape
    G = k.shape[1]
    per = H // G
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        if head_scale is not None:
            s = s * head_scale[h]
        s = s.masked_fill(~mask, float("-inf"))
        if sink:
            m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
            e = torch.exp(s - m)
            p = e / (torch.exp(-m) + e.sum(-1, keepdim=True))
        else:
            p = torch.softmax(s, -1)
        out[:, h] = p @ v[:, g]
    return out


def mixer_attention(h, w, pre, m, eps):
    """Pair-layout rotary, unit RMS norm of q and k per head after the turn,
    sliding window with kept first tokens."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[pre + "q"]).view(T, H, D)
    k = linear(h, w[pre + "k"]).view(T, G, D)
    v = linear(h, w[pre + "v"]).view(T, G, Dv)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot, h.dtype)
        q = rotate(q, pos, f, int(rot["dims"]), "pairs")
        k = rotate(k, pos, f, int(rot["dims"]), "pairs")
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    mask = m.get("mask")
    vis = visible(T, mask["size"] if mask else None,
                  mask.get("keep_first", 0) if mask else 0)
    o = attend(q, k, v, m["scale"], vis)
    return linear(o.reshape(T, H * Dv), w[pre + "o"])


def mixer_attention_2(h, w, pre, m, eps):
    """No positions, values are the keys, a sink of score 0, sigmoid output
    gate read from the mixer input."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = linear(h, w[pre + "q"]).view(T, H, D)
    k = linear(h, w[pre + "k"]).view(T, G, D)
    mask = m.get("mask")
    vis = visible(T, mask["size"] if mask else None,
                  mask.get("keep_first", 0) if mask else 0)
    o = attend(q, k, k, m["scale"], vis, sink=True).reshape(T, H * D)
    o = o * torch.sigmoid(linear(h, w[pre + "g"]))
    return linear(o, w[pre + "o"])


def mixer_attention_3(h, w, pre, m, eps):
    """Biased projections, half-layout rotary, a score multiplier per head,
    every earlier key visible."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[pre + "q"], w[pre + "q.b"]).view(T, H, D)
    k = linear(h, w[pre + "k"], w[pre + "k.b"]).view(T, G, D)
    v = linear(h, w[pre + "v"], w[pre + "v.b"]).view(T, G, Dv)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot, h.dtype)
        q = rotate(q, pos, f, int(rot["dims"]), "halves")
        k = rotate(k, pos, f, int(rot["dims"]), "halves")
    o = attend(q, k, v, m["scale"], visible(T, None, 0),
               head_scale=w[pre + "temp"])
    return linear(o.reshape(T, H * Dv), w[pre + "o"])


MIXERS = {"attention": mixer_attention, "attention_2": mixer_attention_2,
          "attention_3": mixer_attention_3}


# ---- feed-forwards ----------------------------------------------------------
def polynorm(z, coef, eps):
    a, b, c, e = [float(t) for t in coef]
    return (a * rms_unit(z, eps) + b * rms_unit(z * z, eps)
            + c * rms_unit(z * z * z, eps) + e)


def ff_dense(h, w, pre, mlp, eps):
    return linear(polynorm(linear(h, w[pre + "up"]), w[pre + "act"], eps),
                  w[pre + "down"])


def gated_expert(h, w, pre):
    return linear(silu(linear(h, w[pre + "gate"])) * linear(h, w[pre + "up"]),
                  w[pre + "down"])


def route(h, w, pre, r):
    """Returns (ids [T, top], weights [T, top]) over experts + identity
    experts (the latter have the highest indices)."""
    z = linear(h, w[pre + "router"])
    s = torch.softmax(z, -1)
    T, n = s.shape
    choice = s + w[pre + "correction"] if pre + "correction" in w else s.clone()
    g = r.get("groups")
    if g and g["count"] > 1:
        size = n // g["count"]
        gs = choice.view(T, g["count"], size).max(-1).values
        best = gs.topk(g["keep"], -1).indices
        ok = torch.zeros(T, g["count"], dtype=torch.bool).scatter(1, best, True)
        choice = choice.view(T, g["count"], size).masked_fill(
            ~ok[:, :, None], float("-inf")).reshape(T, n)
    ids = choice.topk(r["top"], -1).indices
    wt = s.gather(1, ids)
    return ids, wt / (wt.sum(-1, keepdim=True) + 1e-20)


def ff_moe(h, w, pre, mlp, eps):
    r = mlp["router"]
    ids, wt = route(h, w, pre, r)
    E = r["experts"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j, a in zip(ids[t].tolist(), wt[t]):
            y = h[t] if j >= E else gated_expert(h[t:t + 1], w,
                                                 f"{pre}e{j}.")[0]
            out[t] += a * y
    if mlp.get("shared"):
        out = out + gated_expert(h, w, pre + "shared.")
    return out


def feed_forward(h, w, pre, mlp, eps):
    if mlp["kind"] == "dense":
        return ff_dense(h, w, pre, mlp, eps)
    return ff_moe(h, w, pre, mlp, eps)


# ---- the stack --------------------------------------------------------------
def token_side(x, tokens, w, pre, index, dim, mult, eps):
    e = w["side.embed"][tokens][:, index * dim:(index + 1) * dim]
    g = gelu_tanh(linear(x, w[pre + "side.gate"])) * e
    y = linear(g, w[pre + "side.proj"])
    return x + mult * rms_unit(y, eps) * w[pre + "side.norm"]


def run_layer(x, tokens, cfg, w, i):
    lc, eps = cfg["layers"][i], cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    p = f"l{i}."
    y = MIXERS[lc["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.",
                           lc["mixer"], eps)
    x = x + mult * rms_norm(y, w[p + "norm1b"], eps)
    if lc.get("mlp"):
        y = feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.",
                         lc["mlp"], eps)
        x = x + mult * rms_norm(y, w[p + "norm2b"], eps)
    side = cfg.get("token_side")
    if side:
        x = token_side(x, tokens, w, p, i, side["dim"], mult, eps)
    return x


def forward(cfg, weights, tokens, dtype=torch.float64):
    """-> (logits [T, vocab], residual after every layer run [runs, T, W])."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v)
         for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    e = w["embed"][tokens]
    x = e
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    start, stop, times = (lp["start"], lp["stop"], lp["times"]) if lp \
        else (0, 0, 1)
    after = []
    for i in range(start):
        x = run_layer(x, tokens, cfg, w, i)
        after.append(x)
    for t in range(times if stop > start else 0):
        if t > 0:
            x = x + e
        x = x + w["loop.step"][t]
        for i in range(start, stop):
            x = run_layer(x, tokens, cfg, w, i)
            after.append(x)
    for i in range(stop, n):
        x = run_layer(x, tokens, cfg, w, i)
        after.append(x)
    hid = rms_norm(x, w["final.norm"], cfg["norm"]["eps"])
    return hid @ w["embed"].T, torch.stack(after)


# ---- test models: configurations, random checkpoints, model folders ---------
def attn(kind="attention", heads=4, kv_heads=2, dim=8, vdim=8, dims=4,
         base=100.0, scaling=None, size=5, keep_first=2, scale=None, mlp=12):
    """One layer entry. mlp: int = dense feed-forward of that size, dict =
    as given, None = none. size None = no mask."""
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
             scale=scale if scale is not None else dim ** -0.5)
    if kind != "attention_2" and dims:
        m["rot"] = dict(base=base, dims=dims)
        if scaling:
            m["rot"]["scaling"] = scaling
    if kind != "attention_3" and size is not None:
        m["mask"] = dict(size=size, keep_first=keep_first)
    if kind == "attention_2":
        m["vdim"] = dim
    if isinstance(mlp, int):
        mlp = dict(kind="dense", ff=mlp)
    return dict(type=kind, mixer=m, mlp=mlp)


def moe(ff=6, experts=4, top=2, identity=2, groups=(3, 2), shared=5):
    r = dict(experts=experts, top=top, identity=identity)
    if groups:
        r["groups"] = dict(count=groups[0], keep=groups[1])
    d = dict(kind="moe", expert=dict(ff=ff), router=r)
    if shared:
        d["shared"] = dict(ff=shared)
    return d


def make_config(width=24, vocab=50, eps=1e-5, mult=0.4, side=3, loop=None,
                layers=None):
    d = dict(architecture="Gararax", vocab=vocab, width=width,
             norm=dict(eps=eps), residual_mult=mult,
             layers=layers or [attn("attention_2"), attn("attention_3"),
                               attn("attention")])
    if side:
        d["token_side"] = dict(dim=side)
    if loop:
        d["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return d


def make_weights(cfg, seed=0, gain=1.0):
    """Random bf16-representable weights (fp32 tensors) for a config."""
    g = torch.Generator().manual_seed(seed)
    W, n = cfg["width"], len(cfg["layers"])

    def rnd(*shape, std=None):
        std = std if std is not None else gain / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def near_one(k, spread=0.2):
        return (1.0 + spread * torch.randn(k, generator=g)).bfloat16().float()

    out = {"embed": rnd(cfg["vocab"], W, std=1.0), "final.norm": near_one(W)}
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        out["side.embed"] = rnd(cfg["vocab"], n * side, std=1.0)
    lp = cfg.get("loop")
    if lp and lp["stop"] > lp["start"]:
        out["loop.step"] = rnd(lp["times"], W, std=0.5)
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        mc, m = lc["mixer"], p + "mix."
        H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        for nm in ("norm1", "norm1b"):
            out[p + nm] = near_one(W)
        # queries and keys large enough for a peaked softmax
        out[m + "q"], out[m + "k"] = rnd(H * D, W, std=1.5 / math.sqrt(W)), \
            rnd(G * D, W, std=1.5 / math.sqrt(W))
        if lc["type"] != "attention_2":
            out[m + "v"] = rnd(G * Dv, W)
        else:
            out[m + "g"] = rnd(H * Dv, W)
        if lc["type"] == "attention_3":
            out[m + "q.b"], out[m + "k.b"] = rnd(H * D, std=0.3), \
                rnd(G * D, std=0.3)
            out[m + "v.b"] = rnd(G * Dv, std=0.3)
            out[m + "temp"] = near_one(H, 0.4)
        out[m + "o"] = rnd(W, H * Dv)
        mlp, f = lc.get("mlp"), p + "mlp."
        if mlp:
            for nm in ("norm2", "norm2b"):
                out[p + nm] = near_one(W)
            if mlp["kind"] == "dense":
                out[f + "up"], out[f + "down"] = rnd(mlp["ff"], W), \
                    rnd(W, mlp["ff"])
                out[f + "act"] = rnd(4, std=0.7)
            else:
                r = mlp["router"]
                n_all = r["experts"] + r.get("identity", 0)
                out[f + "router"] = rnd(n_all, W, std=2.0 / math.sqrt(W))
                # corrections comparable to the scores, of both signs
                out[f + "correction"] = rnd(n_all, std=0.5 / n_all)
                ff = mlp["expert"]["ff"]
                for j in range(r["experts"]):
                    e = f"{f}e{j}."
                    out[e + "gate"], out[e + "up"] = rnd(ff, W), rnd(ff, W)
                    out[e + "down"] = rnd(W, ff)
                if mlp.get("shared"):
                    sf = mlp["shared"]["ff"]
                    out[f + "shared.gate"] = rnd(sf, W)
                    out[f + "shared.up"] = rnd(sf, W)
                    out[f + "shared.down"] = rnd(W, sf)
        if side:
            out[p + "side.gate"], out[p + "side.proj"] = rnd(side, W), \
                rnd(W, side)
            out[p + "side.norm"] = near_one(W)
    return out


def write_safetensors(path, tensors):
    """bf16 file: 8-byte header length, JSON header, raw data."""
    import json
    import struct
    header, blobs, at = {}, [], 0
    for name, t in tensors.items():
        raw = t.to(torch.bfloat16).contiguous().view(torch.int16).numpy() \
            .tobytes()
        header[name] = dict(dtype="BF16", shape=list(t.shape),
                            data_offsets=[at, at + len(raw)])
        blobs.append(raw)
        at += len(raw)
    js = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(js)))
        f.write(js)
        for b in blobs:
            f.write(b)


def write_model_dir(folder, cfg, weights):
    import json
    import os
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return folder


def rel_err(got, want):
    """Per row: rms of the mean-free difference over the rms of `want`."""
    got, want = got.to(torch.float64), want.to(torch.float64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return torch.sqrt((d ** 2).mean(-1)) / torch.sqrt((ref ** 2).mean())
