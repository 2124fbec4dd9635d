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
    sink = W("sink")                                                     # [H]
    mx = torch.maximum(s.max(-1).values, sink[:, None])
    e = torch.exp(s - mx[..., None])
    p = e / (e.sum(-1) + torch.exp(sink[:, None] - mx))[..., None]       # the sink takes weight and gives nothing
    o = torch.einsum("hij,jhv->ihv", p, v).reshape(T, H * Dv)
    o = o * torch.sigmoid(h @ W("g").T)
    return o @ W("o").T


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
    decay = torch.tensor([float(a) for a in m["decay"]], dtype=F64)
    S = torch.zeros(H, D, Dv, dtype=F64)
    o = torch.empty(T, H, Dv, dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms_unit(o, eps).reshape(T, H * Dv)
    g = h @ W("g").T
    out = (o * (g * torch.sigmoid(g))) @ W("o").T
    return (out, S) if return_state else out


def dense_ff(h, W, mlp: dict):
    L = float(mlp["limit"])
    g = (h @ W("gate").T).clamp(max=L)
    u = (h @ W("up").T).clamp(-L, L)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W("down").T


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
