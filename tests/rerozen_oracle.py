"""Plain fp64 oracle of the Rerozen design: one function per mechanism, whole sequences, no cache, no batching.

Written from the design's equations and shares no code with the product path.  Weights are a dict name -> tensor with
the checkpoint's names; a config is the config.json dict.  Notation: T tokens, positions t = 0 .. T-1, H query heads,
G key/value heads, D / Dv key / value sizes per head.
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ small pieces
def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w may be None)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def causal_conv(x, w):
    """y_t = sum_j w[:, j] x_(t - taps + 1 + j) per channel; x [T, C], w [C, taps]; zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + w[:, j] * pad[j:j + T]
    return y


def silu(x):
    return x * torch.sigmoid(x)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def rope_freqs(dims, base, scaling=None):
    """(f [dims / 2], table multiplier).  scaling = dict(factor, original, fast, slow): YaRN-style blending."""
    i = torch.arange(dims // 2, dtype=F64)
    f = float(base) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    fac, orig = float(scaling["factor"]), float(scaling["original"])

    def pair_at(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(pair_at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_at(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / fac * ramp + f * (1.0 - ramp), 0.1 * math.log(fac) + 1.0


def rotate(x, pos, f, mult=1.0, sign=1.0):
    """Rotate the first 2 len(f) entries of x [T, heads, n] by pos * f ("rotate half" pairs: i with i + len(f))."""
    n = f.numel()
    a = sign * pos.to(F64)[:, None] * f[None, :]
    c, s = (torch.cos(a) * mult)[:, None, :], (torch.sin(a) * mult)[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], -1)


# ------------------------------------------------------------------ left mixers: chunked rotary attention
def chunk_mask(T, size):
    t = torch.arange(T)
    return (t[None, :] <= t[:, None]) & ((t[None, :] // size) == (t[:, None] // size))


def chunked_softmax_attention(q, k, v, scale, size, sink):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv].  sink: the denominator also holds exp(0) = 1."""
    T, H, _ = q.shape
    G = k.shape[1]
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    vis = chunk_mask(T, size)
    e = torch.exp(s.masked_fill(~vis, -float("inf")))
    den = e.sum(-1, keepdim=True) + (1.0 if sink else 0.0)
    return torch.einsum("hij,jhd->ihd", e / den, v)


def rotary_attention(h, W, p, m, two, eps):
    """The left mixer.  two = False: biases + per-head q/k norms; True: short convolutions, rotated values, a sink."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if two:
        q, k, v = causal_conv(q, W[p + "q.conv"]), causal_conv(k, W[p + "k.conv"]), causal_conv(v, W[p + "v.conv"])
    else:
        q, k, v = q + W[p + "q.b"], k + W[p + "k.b"], v + W[p + "v.b"]
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, Dv)
    if not two:
        q, k = rms_norm(q, W[p + "q.norm"], eps), rms_norm(k, W[p + "k.norm"], eps)
    rot = m["rot"]
    if rot["dims"]:
        f, mult = rope_freqs(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, pos, f, mult), rotate(k, pos, f, mult)
    if two:
        fv, _ = rope_freqs(Dv, rot["base"])
        v = rotate(v, pos, fv)
    o = chunked_softmax_attention(q, k, v, m["scale"], m["mask"]["size"], sink=two)
    if two:
        o = rotate(o, pos, fv, sign=-1.0)
    o = o * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * Dv) @ W[p + "o"].T


# ------------------------------------------------------------------ right mixers: linear attention, decay per channel
def gla_decay(h, W, p, m):
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    return torch.sigmoid(z) ** (1.0 / m["tau"])


def delta_decay(h, W, p, m):
    H, D = m["heads"], m["dim"]
    a = ((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).view(-1, H, D)
    return torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * torch.nn.functional.softplus(a)).reshape(-1, H * D)


def recurrence(q, k, v, g, beta=None, S=None):
    """q, k, g [T, H, D], v [T, H, Dv]; beta [T, H] (delta rule) or None (plain accumulation).  Returns (o, S)."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1], dtype=q.dtype) if S is None else S
    out = []
    for t in range(T):
        S = g[t][:, :, None] * S
        u = v[t] if beta is None else beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out), S


def gated_linear_attention(h, W, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, D) * D ** -0.5
    k, v = (h @ W[p + "k"].T).view(T, H, D), (h @ W[p + "v"].T).view(T, H, Dv)
    o, _ = recurrence(q, k, v, gla_decay(h, W, p, m).view(T, H, D))
    o = rms_norm(o, W[p + "norm"], eps).reshape(T, H * Dv)
    return (o * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def gated_delta_rule(h, W, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, 1), k.repeat_interleave(H // G, 1)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    o, _ = recurrence(q, k, v, delta_decay(h, W, p, m).view(T, H, D), beta)
    o = rms_norm(o, W[p + "norm"], eps).reshape(T, H * Dv)
    return (o * torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T)) @ W[p + "o"].T


# ------------------------------------------------------------------ the model
def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        n = rms_norm(x, W[p + "norm1"], eps)
        h = n + causal_conv(n, W[p + "canon1"])
        two = L["type"] == "parallel_2"
        left = rotary_attention(h, W, p + "mix.left.", m["left"], two, eps)
        right = (gated_delta_rule if two else gated_linear_attention)(h, W, p + "mix.right.", m["right"], eps)
        x = x + m["left_scale"] * left + m["right_scale"] * right
        if L["mlp"] is not None:
            n = rms_norm(x, W[p + "norm2"], eps)
            h = n + causal_conv(n, W[p + "canon2"])
            x = x + gelu_erf(h @ W[p + "mlp.up"].T) @ W[p + "mlp.down"].T
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T * cfg["logit_scale"]


# ------------------------------------------------------------------ configurations and weights for tests
def attention_left(heads, kv_heads, dim, vdim, chunk, rot_dims, base=10000.0, scale=None, conv=None, scaling=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else dim ** -0.5,
             mask=dict(size=chunk), rot=dict(base=base, dims=rot_dims))
    if scaling:
        m["rot"]["scaling"] = scaling
    if conv is not None:
        m["conv"] = conv
    return m


def make_config(width, vocab, layers, taps=4, eps=1e-6, embed_scale=None, logit_scale=0.5):
    """layers: dicts(type, left, right, left_scale, right_scale, ff | None, a_rank, g_rank); ranks are NOT written into
    the config (a checkpoint's tensor shapes carry them) but returned beside it for make_weights."""
    out, ranks = [], []
    for L in layers:
        out.append(dict(type=L["type"], mixer=dict(left=L["left"], right=L["right"], left_scale=L.get("left_scale", 0.7),
                                                   right_scale=L.get("right_scale", 1.3)),
                        mlp=None if not L.get("ff") else dict(kind="dense", ff=L["ff"])))
        ranks.append((L.get("a_rank", 6), L.get("g_rank", 5)))
    cfg = dict(architecture="Rerozen", vocab=vocab, width=width, norm=dict(eps=eps), canon=dict(taps=taps),
               embedding=dict(scale=embed_scale if embed_scale is not None else math.sqrt(width)), logit_scale=logit_scale,
               layers=out)
    return cfg, ranks


def make_weights(cfg, ranks, seed=0):
    """Random bf16 weights with the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    d, taps = cfg["width"], cfg["canon"]["taps"]

    def mat(o, i, s=1.0):
        return torch.randn(o, i, generator=g) * s / math.sqrt(i)

    W = {"embed": torch.randn(cfg["vocab"], d, generator=g) / math.sqrt(d), "final.norm": 1 + 0.1 * torch.randn(d, generator=g),
         "head": mat(cfg["vocab"], d)}
    for i, (L, (ar, gr)) in enumerate(zip(cfg["layers"], ranks)):
        p, a, r = f"l{i}.", L["mixer"]["left"], L["mixer"]["right"]
        two = L["type"] == "parallel_2"
        W[p + "norm1"] = 1 + 0.1 * torch.randn(d, generator=g)
        W[p + "canon1"] = 0.2 * torch.randn(d, taps, generator=g)
        pl, pr = p + "mix.left.", p + "mix.right."
        nq, nk, nv = a["heads"] * a["dim"], a["kv_heads"] * a["dim"], a["kv_heads"] * a["vdim"]
        W.update({pl + "q": mat(nq, d, 2.0), pl + "k": mat(nk, d, 2.0), pl + "v": mat(nv, d), pl + "g": mat(a["heads"], d),
                  pl + "o": mat(d, a["heads"] * a["vdim"])})
        if two:
            for n_, c in (("q", nq), ("k", nk), ("v", nv)):
                W[pl + n_ + ".conv"] = 0.5 * torch.randn(c, a["conv"], generator=g)
        else:
            W.update({pl + "q.b": 0.1 * torch.randn(nq, generator=g), pl + "k.b": 0.1 * torch.randn(nk, generator=g),
                      pl + "v.b": 0.1 * torch.randn(nv, generator=g), pl + "q.norm": 1 + 0.1 * torch.randn(a["dim"], generator=g),
                      pl + "k.norm": 1 + 0.1 * torch.randn(a["dim"], generator=g)})
        H, D, Dv = r["heads"], r["dim"], r["vdim"]
        G = r["kv_heads"] if two else H
        W.update({pr + "q": mat(G * D, d), pr + "k": mat(G * D, d), pr + "v": mat(H * Dv, d), pr + "o": mat(d, H * Dv),
                  pr + "norm": 1 + 0.1 * torch.randn(Dv, generator=g), pr + "a1": mat(ar, d), pr + "a2": mat(H * D, ar, 2.0)})
        if two:
            for n_, c in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                W[pr + n_ + ".conv"] = 0.5 * torch.randn(c, r["conv"], generator=g)
            W.update({pr + "b": mat(H, d), pr + "A_log": torch.rand(H, generator=g) * 2 - 2, pr + "dt_bias": torch.randn(H * D, generator=g),
                      pr + "g1": mat(gr, d), pr + "g2": mat(H * Dv, gr, 2.0)})
        else:
            W.update({pr + "g": mat(H * Dv, d), pr + "a2.b": 1.0 + torch.randn(H * D, generator=g)})
        if L["mlp"] is not None:
            ff = L["mlp"]["ff"]
            W.update({p + "norm2": 1 + 0.1 * torch.randn(d, generator=g), p + "canon2": 0.2 * torch.randn(d, taps, generator=g),
                      p + "mlp.up": mat(ff, d), p + "mlp.down": mat(d, ff)})
    return {k: v.to(torch.bfloat16) for k, v in W.items()}
