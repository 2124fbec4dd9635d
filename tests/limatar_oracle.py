"""Plain float64 oracle of the Limatar design, one function per mechanism (CPU, slow, whole sequences at once).

It shares no code with the product path: weights come as a dict name -> tensor, the configuration as the dict that
a model folder's config.json holds.  Notation: T tokens of ONE sequence at positions 0 .. T-1, d the width.

    norm         x / sqrt(mean(x^2) + eps) * (1 + w)            (weights stored around zero)
    layer        x += norm1b(mixer(norm1(x)));  x += norm2b(ff(norm2(x)))
    latent attn  queries and keys / values through low-rank latents; one rotated key part shared by all heads;
                 softmax whose denominator also holds exp(sink_h); sigmoid output gate
    retention    S_t = a_h S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t  (no softmax), per-head unit RMS, silu gate
    dense ff     g = min(Wg h, L); u = clamp(Wu h, -L, L); Wd (g sigmoid(1.702 g) (u + 1))
    experts      top-k of the router's logits (+ bias), softmax over the chosen, + a shared expert
    loop         layers [start, stop) run `times` times in a row with the same weights
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_zero_centered(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w.to(F64)


def rope_tables(rot: dict, positions: torch.Tensor):
    """cos, sin [T, dims / 2] of the rotation ``rot`` = {base, dims, scaling?}; with ``scaling`` (factor, original,
    fast, slow) the frequencies are blended between f and f / factor over a ramp of the pair index and both tables are
    multiplied by 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def dim_of(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    a = positions.to(F64)[:, None] * f[None, :]
    return torch.cos(a) * mult, torch.sin(a) * mult


def rotate_interleaved(x, cos, sin):
    """x [T, ..., dims]: entry 2i is paired with 2i + 1."""
    u, v = x[..., 0::2], x[..., 1::2]
    shape = [cos.shape[0]] + [1] * (x.dim() - 2) + [cos.shape[1]]
    c, s = cos.view(shape), sin.view(shape)
    out = torch.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


def rotate_half(x, cos, sin):
    """x [T, ..., dims]: entry i is paired with i + dims / 2."""
    n = x.shape[-1] // 2
    u, v = x[..., :n], x[..., n:]
    shape = [cos.shape[0]] + [1] * (x.dim() - 2) + [cos.shape[1]]
    c, s = cos.view(shape), sin.view(shape)
    return torch.cat([u * c - v * s, v * c + u * s], -1)


def sink_softmax(s, sink):
    """Softmax over the last axis of s [H, ..., keys] whose denominator also holds exp(sink_h): the sink takes weight
    and gives nothing (rows do not sum to one)."""
    sk = sink.view([-1] + [1] * (s.dim() - 2))
    mx = torch.maximum(s.max(-1).values, sk)
    e = torch.exp(s - mx[..., None])
    return e / (e.sum(-1) + torch.exp(sk - mx))[..., None]


def latent_attention(h, W: Callable[[str], torch.Tensor], m: dict, eps: float):
    """h [T, d] -> [T, d].  ``W(name)`` gives the mixer's tensor '.name' in float64."""
    T = h.shape[0]
    H, D, R, Dv, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T)
    cos, sin = rope_tables(m["rot"], pos)
    cq = norm_plain(h @ W("dq").T, W("dq.norm"), eps)
    q = (cq @ W("uq").T).view(T, H, D + R)
    q_nope, q_rot = q[..., :D], rotate_interleaved(q[..., D:], cos, sin)
    dkv = h @ W("dkv").T
    c = norm_plain(dkv[:, :C], W("dkv.norm"), eps)
    k_rot = rotate_interleaved(dkv[:, C:], cos, sin)                     # [T, R], one for all heads
    k_nope = (c @ W("uk").T).view(T, H, D)
    v = (c @ W("uv").T).view(T, H, Dv)
    s = (torch.einsum("ihd,jhd->hij", q_nope, k_nope) + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * float(m["scale"])
    s = s.masked_fill(pos[None, :, None] < pos[None, None, :], -math.inf)
    p = sink_softmax(s, W("sink"))
    o = torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * Dv)
    o = o * torch.sigmoid(h @ W("g").T)
    return o @ W("o").T


def retention_scan(q, k, v, decay, S=None):
    """q, k [T, H, D], v [T, H, Dv] -> (o [T, H, Dv], final state [H, D, Dv]): S <- a_h S + k v^T, o = S^T q."""
    T, H, D = q.shape
    a = torch.tensor(list(decay), dtype=F64)[:, None, None]
    S = torch.zeros(H, D, v.shape[-1], dtype=F64) if S is None else S.clone()
    o = torch.empty(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        S = a * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def retention(h, W, m: dict, eps: float, return_state: bool = False):
    """h [T, d] -> [T, d]; the recurrence token by token."""
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    rd = int(m["rot"]["dims"])
    cos, sin = rope_tables(m["rot"], torch.arange(T))
    q = (h @ W("q").T).view(T, H, D).clone()
    k = (h @ W("k").T).view(T, H, D).clone()
    v = (h @ W("v").T).view(T, H, Dv)
    q[..., :rd] = rotate_half(q[..., :rd], cos, sin)
    k[..., :rd] = rotate_half(k[..., :rd], cos, sin)
    k = k * D ** -0.5
    o, S = retention_scan(q, k, v, [float(a) for a in m["decay"]])
    o = rms_unit(o, eps).reshape(T, H * Dv)
    g = h @ W("g").T
    out = (o * (g * torch.sigmoid(g))) @ W("o").T
    return (out, S) if return_state else out


def clamped_unit(g, u, limit: float):
    g, u = g.clamp(max=limit), u.clamp(-limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def dense_ff(h, W, mlp: dict):
    return clamped_unit(h @ W("gate").T, h @ W("up").T, float(mlp["limit"])) @ W("down").T


def gated_expert(h, gate, up, down):
    z = h @ gate.T
    return (z * torch.sigmoid(z) * (h @ up.T)) @ down.T


def route(h, W, mlp: dict):
    """(ids [T, top], weights [T, top]): the largest logits, softmax over the chosen only."""
    z = h @ W("router").T + W("router.b")
    top = torch.topk(z, int(mlp["router"]["top"]), dim=-1)
    return top.indices, torch.softmax(top.values, -1)


def moe_ff(h, W, mlp: dict):
    ids, w = route(h, W, mlp)
    out = torch.zeros_like(h)
    for e in range(int(mlp["router"]["experts"])):
        t, j = (ids == e).nonzero(as_tuple=True)
        if t.numel():
            y = gated_expert(h[t], W(f"e{e}.gate"), W(f"e{e}.up"), W(f"e{e}.down"))
            out.index_add_(0, t, y * w[t, j][:, None])
    if mlp.get("shared"):
        out = out + gated_expert(h, W("shared.gate"), W("shared.up"), W("shared.down"))
    return out


def layer_runs(cfg: dict) -> List[int]:
    """Layer indices in execution order (the looped span repeated in a row)."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg: dict, sd: Dict[str, torch.Tensor], tokens, streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; ``streams`` collects the residual after every layer run."""
    eps = float(cfg["norm"]["eps"])

    def w(name):
        return sd[name].to(F64)

    x = norm_zero_centered(w("embed")[torch.as_tensor(tokens, dtype=torch.long)], w("embed.norm"), eps)
    for li in layer_runs(cfg):
        L, p = cfg["layers"][li], f"l{li}."
        mix = latent_attention if L["type"] == "latent_attention" else retention
        if L["type"] not in ("latent_attention", "retention"):
            raise ValueError(L["type"])
        y = mix(norm_zero_centered(x, w(p + "norm1"), eps), lambda n: w(p + "mix." + n), L["mixer"], eps)
        x = x + norm_zero_centered(y, w(p + "norm1b"), eps)
        if L.get("mlp") is not None:
            ff = dense_ff if L["mlp"]["kind"] == "dense" else moe_ff
            y = ff(norm_zero_centered(x, w(p + "norm2"), eps), lambda n: w(p + "mlp." + n), L["mlp"])
            x = x + norm_zero_centered(y, w(p + "norm2b"), eps)
        if streams is not None:
            streams.append(x.clone())
    return norm_zero_centered(x, w("final.norm"), eps) @ w("embed").T


# ------------------------------------------------------------------ small configurations and random weights for tests
def latent_layer(heads, dim, rot_dim, vdim, q_rank, kv_rank, mlp, scale=None, base=5000.0, scaling=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": rot}}


def retention_layer(heads, dim, vdim, mlp, rot_dims=None, base=3000.0, decay=None):
    decay = decay or [1.0 - 2.0 ** (-2 - 1.5 * h) for h in range(heads)]
    return {"type": "retention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                      "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims}}}


def dense(ff, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def make_config(width, vocab, layers, loop=None, eps=1e-5):
    cfg = {"architecture": "Limatar", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bf16 tensors under the names a checkpoint of the design uses."""
    g = torch.Generator().manual_seed(seed)
    d, V = int(cfg["width"]), int(cfg["vocab"])

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, s=0.1, mean=0.0):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    W = {"embed": (0.25 * torch.randn(V, d, generator=g)).to(torch.bfloat16), "embed.norm": vec(d), "final.norm": vec(d)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        W[p + "norm1"], W[p + "norm1b"] = vec(d), vec(d)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "latent_attention":
            R, C, Cq = m["rot_dim"], m["kv_rank"], m["q_rank"]
            W[p + "mix.dq"], W[p + "mix.dq.norm"], W[p + "mix.uq"] = mat(Cq, d), vec(Cq, mean=1.0), mat(H * (D + R), Cq, 2.0)
            W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = mat(C + R, d), vec(C, mean=1.0)
            W[p + "mix.uk"], W[p + "mix.uv"], W[p + "mix.sink"] = mat(H * D, C, 2.0), mat(H * Dv, C), vec(H, 1.0)
        else:
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = mat(H * D, d), mat(H * D, d), mat(H * Dv, d)
        W[p + "mix.g"], W[p + "mix.o"] = mat(H * Dv, d), mat(d, H * Dv)
        e = L.get("mlp")
        if e is None:
            continue
        W[p + "norm2"], W[p + "norm2b"] = vec(d), vec(d)
        if e["kind"] == "dense":
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = mat(e["ff"], d, 2.0), mat(e["ff"], d, 2.0), mat(d, e["ff"])
        else:
            ff = e["expert"]["ff"]
            W[p + "mlp.router"], W[p + "mlp.router.b"] = mat(e["router"]["experts"], d, 3.0), vec(e["router"]["experts"], 0.5)
            for x in range(e["router"]["experts"]):
                W[f"{p}mlp.e{x}.gate"], W[f"{p}mlp.e{x}.up"], W[f"{p}mlp.e{x}.down"] = mat(ff, d), mat(ff, d), mat(d, ff)
            if e.get("shared"):
                sf = e["shared"]["ff"]
                W[p + "mlp.shared.gate"], W[p + "mlp.shared.up"], W[p + "mlp.shared.down"] = mat(sf, d), mat(sf, d), mat(d, sf)
    return W
