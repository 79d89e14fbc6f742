"""Slow, plain fp64 oracle for the Tosipel decoder — one function per
mechanism, written from the equations, sharing nothing with the package.

  rms                   x / sqrt(mean(x^2) + eps)
  post norm             x <- x + rms(sublayer(x)) * (1 + w): the sublayer
                        reads the residual itself, only its output is normed
  rotary (halves)       entry i of a head is paired with entry i + dims/2;
                        (u, v) -> (u c - v s, v c + u s), angle p * f_i,
                        f_i = base^(-2i/dims); entries past `dims` untouched
  windowed attention    rms over the WHOLE q (and k) projection before the
                        split into heads; keys j with 0 <= i - j < size;
                        softmax whose denominator also holds exp(sink_h);
                        head output times sigmoid of one gate number per head
  latent attention      q through a normed low-rank latent; keys and values
                        are linear images of one normed latent per token;
                        causal softmax, no positions
  gated delta rule      short causal convolution + silu on q, k, v; unit q
                        and k per head; S <- g S; u = beta (v - S^T k);
                        S <- S + k u^T; o = S^T q; per-head rms, silu gate
  feed-forward          down(gelu_tanh(gate h) * up h)
  shared weights        a layer may use another layer's tensors, with a cache
                        of its own

Also config / checkpoint generators and a minimal safetensors writer so tests
can hand the engine a model folder of their own making.
"""
import json
import math
import os
import struct

import torch

F64 = torch.float64


# ---------------------------------------------------------------- mechanisms
def o_rms(x, eps):
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)


def o_sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def o_silu(x):
    return x * o_sigmoid(x)


def o_softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(
        x, max=30.0))))


def o_gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def o_rotate_halves(vec, pos, rot):
    """vec 1-D (one head): entry i turns together with entry i + dims/2."""
    out = vec.clone()
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, v = float(vec[i]), float(vec[i + half])
        out[i] = u * c - v * s
        out[i + half] = v * c + u * s
    return out


def o_conv(u, w):
    """u [T, C], w [C, taps]: the last column multiplies the current row,
    rows before the start are zero."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * u[src]
    return out


def o_attend(q, keys, values, scale, sink=None):
    """One query vector against the keys it sees: softmax(scale q.k) v,
    with exp(sink) as one more term of the denominator when given."""
    s = (keys @ q) * scale
    m = float(s.max()) if sink is None else max(float(s.max()), float(sink))
    e = torch.exp(s - m)
    den = e.sum() + (0.0 if sink is None else math.exp(float(sink) - m))
    return (e / den) @ values


def o_delta_core(q, k, v, b, a, A_log, dt_bias, S=None):
    """q, k [T, G, D] and v [T, H, Dv] after convolution and silu, b and a
    [T, H] as projected. Returns the read-outs [T, H, Dv] and the state
    [H, D, Dv] after the last token."""
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    per = H // G
    q = q / torch.sqrt((q ** 2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k ** 2).sum(-1, keepdim=True) + 1e-6)
    beta = o_sigmoid(b)
    g = torch.exp(-torch.exp(A_log) * o_softplus(a + dt_bias))
    S = torch.zeros(H, D, Dv, dtype=F64) if S is None else S.clone()
    o = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        for n in range(H):
            kk, qq = k[t, n // per], q[t, n // per]
            S[n] = g[t, n] * S[n]
            u = beta[t, n] * (v[t, n] - S[n].T @ kk)
            S[n] = S[n] + torch.outer(kk, u)
            o[t, n] = S[n].T @ qq
    return o, S


def o_window_attention(Wt, p, mc, h, eps):
    T = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    per = H // G
    q = o_rms(h @ Wt[p + "q"].T, eps) * Wt[p + "q.norm"]
    k = o_rms(h @ Wt[p + "k"].T, eps) * Wt[p + "k.norm"]
    v = (h @ Wt[p + "v"].T).view(T, G, Dv)
    q, k = q.view(T, H, D).clone(), k.view(T, G, D).clone()
    rot = mc.get("rot")
    if rot and rot.get("dims"):
        for t in range(T):
            for a in range(H):
                q[t, a] = o_rotate_halves(q[t, a], t, rot)
            for a in range(G):
                k[t, a] = o_rotate_halves(k[t, a], t, rot)
    gate = o_sigmoid(h @ Wt[p + "g"].T)                      # [T, H]
    size = int(mc["mask"]["size"])
    out = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        lo = max(0, t - size + 1)
        for a in range(H):
            kv = a // per
            out[t, a] = o_attend(q[t, a], k[lo:t + 1, kv], v[lo:t + 1, kv],
                                 mc["scale"], Wt[p + "sink"][a]) * gate[t, a]
    return out.reshape(T, H * Dv) @ Wt[p + "o"].T


def o_latent_attention(Wt, p, mc, h, eps):
    T = h.shape[0]
    H, D, Dv = mc["heads"], mc["dim"], mc["vdim"]
    cq = o_rms(h @ Wt[p + "dq"].T, eps) * Wt[p + "dq.norm"]
    q = (cq @ Wt[p + "uq"].T).view(T, H, D)
    c = o_rms(h @ Wt[p + "dkv"].T, eps) * Wt[p + "dkv.norm"]
    k = (c @ Wt[p + "uk"].T).view(T, H, D)
    v = (c @ Wt[p + "uv"].T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        for a in range(H):
            out[t, a] = o_attend(q[t, a], k[:t + 1, a], v[:t + 1, a],
                                 mc["scale"])
    return out.reshape(T, H * Dv) @ Wt[p + "o"].T


def o_delta(Wt, p, mc, h, eps):
    T = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = o_silu(o_conv(h @ Wt[p + "q"].T, Wt[p + "q.conv"])).view(T, G, D)
    k = o_silu(o_conv(h @ Wt[p + "k"].T, Wt[p + "k.conv"])).view(T, G, D)
    v = o_silu(o_conv(h @ Wt[p + "v"].T, Wt[p + "v.conv"])).view(T, H, Dv)
    o, _ = o_delta_core(q, k, v, h @ Wt[p + "b"].T, h @ Wt[p + "a"].T,
                        Wt[p + "A_log"], Wt[p + "dt_bias"])
    o = o_rms(o, eps) * Wt[p + "norm"]
    o = o.reshape(T, H * Dv) * o_silu(h @ Wt[p + "g"].T)
    return o @ Wt[p + "o"].T


def o_mixer(Wt, p, lc, h, eps):
    fn = {"attention": o_window_attention,
          "latent_attention": o_latent_attention, "delta": o_delta}
    return fn[lc["type"]](Wt, p + "mix.", lc["mixer"], h, eps)


def o_ff(Wt, p, h):
    return (o_gelu_tanh(h @ Wt[p + "gate"].T) * (h @ Wt[p + "up"].T)) \
        @ Wt[p + "down"].T


def o_forward(cfg, Wt, tokens):
    """-> logits [T, vocab], residual after every layer [layers, T, W]."""
    eps = cfg["norm"]["eps"]
    x = Wt["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    after = []
    for i, lc in enumerate(cfg["layers"]):
        j = lc.get("weights_of")
        p = f"l{i if j is None else j}."
        x = x + o_rms(o_mixer(Wt, p, lc, x, eps), eps) * (1 + Wt[p + "norm1"])
        if lc.get("mlp") is not None:
            x = x + o_rms(o_ff(Wt, p + "mlp.", x), eps) * (1 + Wt[p + "norm2"])
        after.append(x)
    x = o_rms(x, eps) * (1 + Wt["final.norm"])
    return x @ Wt["head"].T, torch.stack(after)


# ------------------------------------------------------- configs and weights
def attn_layer(heads=4, kv_heads=2, dim=8, vdim=6, dims=4, base=100.0,
               scale=None, size=5, mlp=10, weights_of=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                 mask=dict(size=size), rot=dict(base=base, dims=dims),
                 scale=scale if scale is not None else dim ** -0.5)
    out = {"type": "attention", "mixer": mixer,
           "mlp": None if mlp is None else dict(kind="dense", ff=mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def lat_layer(heads=2, dim=6, vdim=5, kv_rank=12, q_rank=10, scale=None,
              mlp=10, weights_of=None):
    mixer = dict(heads=heads, dim=dim, vdim=vdim, kv_rank=kv_rank,
                 q_rank=q_rank,
                 scale=scale if scale is not None else dim ** -0.5)
    out = {"type": "latent_attention", "mixer": mixer,
           "mlp": None if mlp is None else dict(kind="dense", ff=mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def delta_layer(heads=4, kv_heads=2, dim=6, vdim=5, conv=3, mlp=None,
                weights_of=None):
    out = {"type": "delta",
           "mixer": dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                         conv=conv),
           "mlp": None if mlp is None else dict(kind="dense", ff=mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def make_config(width=24, vocab=50, eps=1e-5, embed_scale=3.0, layers=None):
    return dict(architecture="Tosipel", vocab=vocab, width=width,
                embedding=dict(scale=embed_scale), norm=dict(eps=eps),
                layers=layers or [delta_layer(), attn_layer(), lat_layer()])


def make_weights(cfg, seed=0, gain=1.0):
    """Random bf16-representable weights (fp32 tensors) for a config."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rnd(*shape, std=None):
        std = std if std is not None else gain / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def near_one(n, spread=0.2):
        return (1.0 + spread * torch.randn(n, generator=g)).bfloat16().float()

    out = {"embed": rnd(cfg["vocab"], W, std=1.0 / cfg["embedding"]["scale"]),
           "final.norm": rnd(W, std=0.2), "head": rnd(cfg["vocab"], W)}
    for i, lc in enumerate(cfg["layers"]):
        if lc.get("weights_of") is not None:
            continue
        p = f"l{i}."
        out[p + "norm1"] = rnd(W, std=0.2)
        mc, m = lc["mixer"], p + "mix."
        if lc["type"] == "attention":
            H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
            out[m + "q"], out[m + "k"] = rnd(H * D, W), rnd(G * D, W)
            out[m + "v"] = rnd(G * Dv, W)
            out[m + "q.norm"], out[m + "k.norm"] = near_one(H * D), \
                near_one(G * D)
            out[m + "sink"] = rnd(H, std=1.0)
            out[m + "g"], out[m + "o"] = rnd(H, W), rnd(W, H * Dv)
        elif lc["type"] == "latent_attention":
            H, D, Dv = mc["heads"], mc["dim"], mc["vdim"]
            rq, rk = mc["q_rank"], mc["kv_rank"]
            out[m + "dq"], out[m + "dq.norm"] = rnd(rq, W), near_one(rq)
            out[m + "uq"] = rnd(H * D, rq)
            out[m + "dkv"], out[m + "dkv.norm"] = rnd(rk, W), near_one(rk)
            out[m + "uk"], out[m + "uv"] = rnd(H * D, rk), rnd(H * Dv, rk)
            out[m + "o"] = rnd(W, H * Dv)
        else:
            H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                out[m + n] = rnd(rows, W)
                out[f"{m}{n}.conv"] = rnd(rows, mc["conv"], std=0.6)
            out[m + "b"], out[m + "a"] = rnd(H, W), rnd(H, W)
            out[m + "A_log"] = (rnd(H, std=0.7) - 1.0).bfloat16().float()
            out[m + "dt_bias"] = rnd(H, std=1.0)
            out[m + "norm"] = near_one(Dv)
            out[m + "g"], out[m + "o"] = rnd(H * Dv, W), rnd(W, H * Dv)
        if lc.get("mlp") is not None:
            out[p + "norm2"] = rnd(W, std=0.2)
            ff = lc["mlp"]["ff"]
            out[p + "mlp.gate"], out[p + "mlp.up"] = rnd(ff, W), rnd(ff, W)
            out[p + "mlp.down"] = rnd(W, ff)
    # what the file holds is what the oracle sees
    return {k: v.bfloat16().float() for k, v in out.items()}


def write_safetensors(path, tensors):
    header, blobs, off = {}, [], 0
    for name, t in tensors.items():
        raw = t.to(torch.bfloat16).contiguous().view(torch.int16).numpy() \
            .tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape),
                        "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


def write_model_dir(folder, cfg, weights):
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return folder


def as_f64(weights):
    return {k: v.to(F64) for k, v in weights.items()}


def rel_err(got, want):
    """Per row: rms of the mean-free difference over the rms of `want`."""
    got, want = got.to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return torch.sqrt((d ** 2).mean(-1)) / torch.sqrt((ref ** 2).mean())
