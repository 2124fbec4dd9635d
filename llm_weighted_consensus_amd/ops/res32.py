"""Python face of the fp32-residual kernel set (``csrc/kernels/res32`` -> ``ops/_res32.so``).

For decoder designs that keep their residual stream, norms, attention scores and cache-write arithmetic in fp32
while the activations between kernels are bf16 (serving) or fp32 (exact mode).  The extension is separate from
``_kernels.so`` so that a model of such a design needs only this one built; it is compiled on first use when
missing (a fresh checkout), and there is no eager-PyTorch fallback.

Cache layout shared with :class:`..models.cache.PagedLayerCache`: per layer K ``[num_blocks, block_size, G*D]``
and V ``[num_blocks, block_size/4, G*Dv, 4]`` (4-token interleaved) as strided views of one pool.
"""
from __future__ import annotations

import importlib
import math
import threading
from typing import Optional

import torch

_K = None
_LOCK = threading.Lock()


def kernels():
    """The loaded ``_res32`` extension; built in-tree first when it is not there."""
    global _K
    if _K is None:
        with _LOCK:
            if _K is None:
                try:
                    _K = importlib.import_module("llm_weighted_consensus_amd.ops._res32")
                except ImportError:
                    from .. import _build

                    _build.build_res32()
                    _K = importlib.import_module("llm_weighted_consensus_amd.ops._res32")
    return _K


def sinpos_inv_freq(d: int, base: float = 10000.0, device="cuda") -> torch.Tensor:
    """base^(-2i/d) for i < ceil(d/2), in float64 (the kernel reduces p * f mod 2 pi in double)."""
    i2 = torch.arange(0, d, 2, dtype=torch.float64)
    return (float(base) ** (-i2 / d)).to(device)


def embed_sinpos(table: torch.Tensor, tokens: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[t] = table[tokens[t]] + s(positions[t]) in fp32, s[2i] = sin(p f_i), s[2i+1] = cos(p f_i)."""
    if out is None:
        out = torch.empty(tokens.numel(), table.shape[1], dtype=torch.float32, device=table.device)
    kernels().embed_sinpos(table, tokens, positions, inv_freq, out)
    return out


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm with weight and bias of fp32 rows (statistics in fp32) -> rows of ``w``'s dtype.  ``rows``
    (int64): normalise only these rows of ``x``, in this order."""
    n = x.shape[0] if rows is None else rows.numel()
    if out is None:
        out = torch.empty(n, x.shape[1], dtype=w.dtype, device=x.device)
    kernels().layernorm(x, rows, w, b, out, float(eps))
    return out


def proj_norm_kv_write(proj: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, head_scale: torch.Tensor,
                       slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, D: int, eps: float,
                       lam: Optional[torch.Tensor] = None, v0: Optional[torch.Tensor] = None, vmode: int = 0,
                       q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From fused projection rows ``[q | k | v | ...]``: q and k each RMS-normalised over their whole projection
    (all heads at once) with plain weights; q scaled per head by ``head_scale`` into an fp32 buffer (returned);
    k and v written into the paged cache at ``slots`` (-1: no write).  ``vmode`` 1 publishes v into ``v0``
    (fp32 [T, nv]); 2 blends v <- (1 - lam) v + lam v0 before the cache write."""
    if q_out is None:
        q_out = torch.empty(proj.shape[0], H * D, dtype=torch.float32, device=proj.device)
    kernels().proj_norm_kv_write(proj, wq, wk, head_scale, lam, v0, int(vmode), slots, q_out, k_cache, v_cache,
                                 int(H), int(D), float(eps))
    return q_out


def xielu(z: torch.Tensor, pq: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """xIELU with the two raw parameters ``pq`` = (p, q): z > 0: softplus(p) z^2 + z/2; else
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2.  ``z`` and ``out`` may be column slices of wider row-dense buffers."""
    kernels().xielu(z, pq, out)
    return out


def residual_add_scaled(x: torch.Tensor, y: torch.Tensor, m: float) -> None:
    """x (fp32) += m * y, in place."""
    kernels().residual_add_scaled(x, y, float(m))


def residual_add_partials(x: torch.Tensor, parts: torch.Tensor, m: float) -> None:
    """x (fp32) += m * parts.sum(0), parts fp32 [S, *x.shape] (the partial products of a split-K GEMM)."""
    kernels().residual_add_partials(x, parts, float(m))


def distance_bias(r1: torch.Tensor, r2: torch.Tensor, window: int) -> torch.Tensor:
    """The table b[h, n] = r1_h ln(1 + r2_h n), n < window (fp32), that the matrix-core kernel reads."""
    n = torch.arange(window, dtype=torch.float32, device=r1.device)
    return (r1.float()[:, None] * torch.log1p(r2.float()[:, None] * n[None, :])).contiguous()


def window_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, positions: torch.Tensor,
                block_tables: torch.Tensor, r1: torch.Tensor, r2: torch.Tensor, window: int, out: torch.Tensor,
                H: int, G: int, cu_q: Optional[torch.Tensor] = None, k_lens: Optional[torch.Tensor] = None,
                max_q: int = 0, bias: Optional[torch.Tensor] = None, cores: Optional[bool] = None,
                sink: Optional[torch.Tensor] = None, values_in_keys: bool = False, chunk: int = 0) -> torch.Tensor:
    """Sliding-window attention over the paged cache with the bias -r1_h ln(1 + r2_h (i - j)); ``q`` fp32
    [T, H*D] pre-scaled; row t reads table row t (``cu_q`` None) or the item whose ``cu_q`` range holds t.
    Over a bf16 cache whose sizes the matrix-core kernels are built for, prompt portions run on the portion kernel
    (it wants ``k_lens``, ``max_q`` and the ``bias`` table of :func:`distance_bias`) and decode rows on the
    split-key decode kernel (``bias``); everything else on the general kernel.  ``cores=True`` with ``bias`` None:
    the matrix-core kernels without a distance bias (r1 = 0: plain causal or windowed softmax attention).
    ``sink`` (fp32 [H]): exp(sink_h) joins head h's softmax denominator; it has no key and no value.
    ``values_in_keys``: the caller guarantees that every token's value row repeats the first Dv entries of its key row
    (a cached latent that is key and value at once); the decode kernel for one wide row (576 / 512) then takes its
    values from the key rows.
    ``chunk`` > 0: positions are cut into chunks of that many, counted from position 0, and a row sees only keys of its
    own chunk (j >= i - i % chunk), besides the window."""
    K = kernels()
    bs = k_cache.shape[1]
    D, Dv = k_cache.shape[2] // G, v_cache.shape[2] // G
    cores = (bias is not None or bool(cores)) and k_cache.dtype == torch.bfloat16 and bs & (bs - 1) == 0
    if cores and cu_q is None and positions.numel() > 0 and K.window_attn_decode_ok(D, Dv, bool(values_in_keys)):
        max_keys = min(int(window), block_tables.shape[1] * k_cache.shape[1], int(chunk) if chunk > 0 else 1 << 30)
        K.window_attn_decode(q, k_cache, v_cache, positions, block_tables, bias, int(window), max_keys, out, int(H), int(G),
                             sink, bool(values_in_keys), int(chunk))
        return out
    if cores and cu_q is not None and k_lens is not None and max_q > 0 and K.window_attn_mfma_ok(D, Dv):
        K.window_attn_mfma(q, k_cache, v_cache, positions, cu_q, k_lens, int(max_q), block_tables, bias, int(window), out,
                           int(H), int(G), sink, int(chunk))
        return out
    K.window_attn(q, k_cache, v_cache, positions, cu_q, block_tables, r1, r2, int(window), out, int(H), int(G), sink,
                  int(chunk))
    return out


def softplus(x: float) -> float:
    return max(x, 0.0) + math.log1p(math.exp(-abs(x)))


# ------------------------------------------------------------------ recurrent state, gated layers, routed experts
class StepItems:
    """A step's rows grouped by sequence for the kernels that carry per-sequence state: item i owns rows
    [cu[i], cu[i+1]) at consecutive positions and the state slot ``slots[i]`` (a decode row is an item of one
    row).  All int32 device tensors; ``row_item[t]`` is the item of row t."""

    def __init__(self, row_item: torch.Tensor, cu: torch.Tensor, slots: torch.Tensor, positions: torch.Tensor,
                 single: bool = False):
        self.row_item, self.cu, self.slots, self.positions = row_item, cu, slots, positions
        self.single = single  # every item is one row: kernels may advance the state in the same pass

    @classmethod
    def rows(cls, slots: torch.Tensor, positions: torch.Tensor) -> "StepItems":
        """Every row its own item (a decode step); built from device tensors only (capturable)."""
        n = positions.numel()
        ar = torch.arange(n + 1, dtype=torch.int32, device=positions.device)
        return cls(ar[:n], ar, slots, positions, single=True)


def conv_hist(x: torch.Tensor, w: torch.Tensor, hist: torch.Tensor, items: StepItems, out: torch.Tensor,
              mode: int = 0, out2: Optional[torch.Tensor] = None, update: bool = True) -> torch.Tensor:
    """Causal convolution over time per channel with the inputs before a portion's first row taken from the
    sequence's slot of ``hist`` (fp32 [slots, taps - 1, C]); ``w`` fp32 [C, taps], last column = the current
    row's.  ``mode`` 0: out = x + conv(x) (``out2``: a copy of x in out's dtype); 1: out = silu(conv(x)); 2: out = conv(x).
    With ``update`` the slot then holds the last taps - 1 inputs after this step."""
    K = kernels()
    fused = bool(update and items.single)  # a decode step: one kernel computes and moves the history on
    K.conv_hist(x, w, hist, items.row_item, items.cu, items.slots, items.positions, out, out2, int(mode), fused)
    if update and not fused:
        K.conv_hist_update(x, hist, items.cu, items.slots, int(w.shape[1]))
    return out


def delta_rule(qkv: torch.Tensor, ba: torch.Tensor, b_off: int, a_off: int, A_log: torch.Tensor, dt_bias: torch.Tensor,
               state: torch.Tensor, items: StepItems, H: int, G: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gated delta rule over a step's items: per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
    with q, k unit vectors per head (q times D^-1/2), beta = sigmoid(ba[:, b_off + h]),
    g = exp(-exp(A_log_h) softplus(ba[:, a_off + h] + dt_bias_h)).  ``qkv`` fp32 [T, 2 G D + H Dv] (after the
    short convolutions; its q and k columns are normalised IN PLACE), ``state`` fp32 [slots, H, D, Dv] (read unless the item starts at position 0, written
    back).  Returns o fp32 [T, H Dv]."""
    if out is None:
        out = torch.empty(qkv.shape[0], H * state.shape[3], dtype=torch.float32, device=qkv.device)
    kernels().delta_rule(qkv, ba, int(b_off), int(a_off), A_log, dt_bias, state, items.cu, items.slots, items.positions,
                         out, int(H), int(G))
    return out


def head_norm_gate(o: torch.Tensor, out: torch.Tensor, H: int, eps: float, w: Optional[torch.Tensor] = None,
                   gate: Optional[torch.Tensor] = None, mode: str = "silu") -> torch.Tensor:
    """out = o / rms(o) per head * w * act(gate); o fp32 [T, H Dv], ``mode`` silu | sigmoid (ignored without gate)."""
    kernels().head_norm_gate(o, gate, w, out, int(H), float(eps), 0 if gate is None else (1 if mode == "silu" else 2))
    return out


def embed_rows(table: torch.Tensor, tokens: torch.Tensor, out: Optional[torch.Tensor] = None,
               scale: float = 1.0) -> torch.Tensor:
    """x[t] = table[tokens[t]] * scale as fp32."""
    if out is None:
        out = torch.empty(tokens.numel(), table.shape[1], dtype=torch.float32, device=table.device)
    kernels().embed_rows(table, tokens, out, float(scale))
    return out


def head_norm_kv_write(proj: torch.Tensor, k_off: int, v_off: int, positions: torch.Tensor, slots: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, G: int, eps: float, scale: float,
                       temp_coef: float = 0.0, temp_every: int = 0, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From fused projection rows (q at column 0, k at ``k_off``, values at ``v_off``; ``v_off == k_off``: the
    keys as projected are the values): q and k divided by their root mean square per head; q times
    ``scale * (1 + temp_coef ln(floor((p + 1) / temp_every) + 1))`` into an fp32 buffer (returned); the normalised k
    and the values into the paged cache at ``slots`` (-1: no write)."""
    D = k_cache.shape[2] // G
    if q_out is None:
        q_out = torch.empty(proj.shape[0], H * D, dtype=torch.float32, device=proj.device)
    kernels().head_norm_kv_write(proj, int(k_off), int(v_off), positions, slots, q_out, k_cache, v_cache, int(H), int(G),
                                 float(eps), float(scale), float(temp_coef), int(temp_every))
    return q_out


def gate_mul(a: torch.Tensor, g: torch.Tensor, mode: str = "sigmoid") -> torch.Tensor:
    """a *= sigmoid(g) (or silu(g)) in place; both may be column slices of row-dense buffers."""
    kernels().gate_mul(a, g, 0 if mode == "sigmoid" else 1)
    return a


def gated_norm_residual(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float,
                        gate_logits: Optional[torch.Tensor] = None, x_cast: Optional[torch.Tensor] = None,
                        next_w: Optional[torch.Tensor] = None) -> None:
    """x (fp32) += z / rms(z) * w with z = y * sigmoid(gate_logits) (z = y without); w fp32.  ``x_cast`` (bf16
    [T, d]) also receives the new x, or with ``next_w`` (fp32 [d]) the next sublayer's input norm of it,
    x / rms(x) * next_w."""
    kernels().gated_norm_residual(x, y, gate_logits, w, x_cast, float(eps), next_w)


def rmsnorm_rows(x: torch.Tensor, w: torch.Tensor, eps: float, dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMS norm of fp32 rows (optionally the gathered ``rows``, int64) with fp32 weight -> ``dtype`` rows."""
    n = x.shape[0] if rows is None else rows.numel()
    out = torch.empty(n, x.shape[1], dtype=dtype, device=x.device)
    kernels().rmsnorm_rows(x, rows, w, out, float(eps))
    return out


def gelu_mul_rows(z: torch.Tensor, table: torch.Tensor, off: int, tokens: torch.Tensor) -> torch.Tensor:
    """gelu_tanh(z[t]) * table[tokens[t], off : off + n] for z [T, n]."""
    out = torch.empty(z.shape[0], z.shape[1], dtype=z.dtype, device=z.device)
    kernels().gelu_mul_rows(z, table, int(off), tokens, out)
    return out


def stack_mix(X: torch.Tensor, coef: torch.Tensor, n: int, out: torch.Tensor) -> torch.Tensor:
    """out = sum_{j < n} coef[j] X[j] over a stack of fp32 streams X [>= n, T, d]."""
    kernels().stack_mix(X, coef, int(n), out)
    return out


def router(z: torch.Tensor, correction: Optional[torch.Tensor], experts: int, top: int,
           bias: Optional[torch.Tensor] = None, renorm: bool = False):
    """Softmax router over all outputs of ``z`` (fp32 [T, NE]) + ``bias``; the ``top`` largest of softmax + correction
    are chosen, weighted by their softmax (``renorm``: divided by the chosen ones' sum, which is the softmax over the
    chosen logits only).  Outputs >= ``experts`` are identity experts.  Returns
    (ids [T, top], w [T, top], row_off [experts + 1], src [T top], row_expert [T top], inv [T top]): expert-major
    row r holds token src[r] for expert row_expert[r]; choice (t, j) is row inv[t top + j], -1 for an identity."""
    return tuple(kernels().router(z, correction, int(experts), int(top), bias, bool(renorm)))


def expert_rows(h: torch.Tensor, src: torch.Tensor, row_expert: torch.Tensor, row_off: torch.Tensor, w_gu: torch.Tensor,
                w_down: torch.Tensor) -> torch.Tensor:
    """Y[r] = W_down[e] (silu(W_gate[e] h) * (W_up[e] h)) for every expert-major row r (fp32 sums, any sizes)."""
    return kernels().expert_rows(h, src, row_expert, row_off, w_gu, w_down)


def moe_combine(Y: torch.Tensor, inv: torch.Tensor, w: torch.Tensor, h: torch.Tensor,
                add: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 [T, d]: sum_j w[t, j] * (Y[inv[t, j]] if inv >= 0 else h[t]) (+ ``add[t]``: a shared expert's rows)."""
    return kernels().moe_combine(Y, inv, w, h, add)


# ------------------------------------------------------------------ rotations, low-rank attention, retention, gated units
def rope_frequencies(dims: int, base: float, scaling: Optional[dict] = None, device="cuda"):
    """(f fp32 [dims / 2], m): the rotation frequencies base^(-2i/dims) and the multiplier of the cos / sin tables.
    ``scaling`` = {factor, original, fast, slow} blends f_i with f_i / factor over a linear ramp of the pair index i
    between the pairs that turn ``fast`` and ``slow`` times within ``original`` positions, and sets
    m = 0.1 ln(factor) + 1.  Computed in float64, rounded once."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    m = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns: float) -> float:
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        m = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device), m


def latent_kv_write(proj: torch.Tensor, Cq: int, C: int, R: int, wq: torch.Tensor, wc: torch.Tensor, freq: torch.Tensor,
                    mult: float, positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    eps: float, cq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Cache side of a low-rank attention layer.  ``proj`` rows = [dq (Cq) | c (C) | key part to rotate (R) | ...]:
    returns cq = dq / rms(dq) * wq ([T, Cq], proj's dtype); writes per token ONE key row [c / rms(c) * wc | rotated
    part * mult | zeros] and the same normalised c as its value row into the paged cache at ``slots`` (-1: no write).
    Rotation: entries (2i, 2i + 1) by the angle position * freq[i]."""
    if cq is None:
        cq = torch.empty(proj.shape[0], Cq, dtype=proj.dtype, device=proj.device)
    kernels().latent_kv_write(proj, int(Cq), int(C), int(R), wq, wc, freq, float(mult), positions, slots, cq, k_cache,
                              v_cache, float(eps))
    return cq


def latent_q_rows(q: torch.Tensor, D: int, R: int, qn: Optional[torch.Tensor], freq: torch.Tensor, mult: float, scale: float,
                  positions: torch.Tensor, H: int, Dk: int) -> torch.Tensor:
    """fp32 query rows [T, H, Dk] of a low-rank attention layer: per head [qn * scale | rot(q[:, D : D + R]) * mult *
    scale | 0], ``qn`` fp32 [H, T, C] = the unrotated query parts times the keys' up-projection; ``qn`` None: the
    unrotated parts themselves (q[:, :D] of every head)."""
    out = torch.empty(q.shape[0], H, Dk, dtype=torch.float32, device=q.device)
    kernels().latent_q_rows(q, int(D), int(R), qn, freq, float(mult), float(scale), positions, out, int(H))
    return out


def latent_expand_write(kv: torch.Tensor, lat: torch.Tensor, rot_off: int, R: int, slots: torch.Tensor, k_cache: torch.Tensor,
                        v_cache: torch.Tensor, H: int, D: int, Dv: int) -> None:
    """Keys and values up-projected from cached latents, written as pages of their own: ``kv`` [N, H D + H Dv], ``lat``
    the tokens' cached rows (their rotated key part at ``rot_off``), ``slots`` int64 [N].  Per token and head the key
    row is [key (D) | rotated part (R) | zeros], the value row [value (Dv) | zeros] (4-token interleaved)."""
    kernels().latent_expand_write(kv, lat, int(rot_off), int(R), slots, k_cache, v_cache, int(H), int(D), int(Dv))


def retention(proj: torch.Tensor, k_off: int, v: torch.Tensor, freq: torch.Tensor, mult: float, rot_dims: int,
              decay: torch.Tensor, state: torch.Tensor, items: StepItems, H: int,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Retention over a step's items: per head S <- a_h S + k v^T, o = S^T q (no softmax, no denominator).  q (columns
    0 ..) and k (columns ``k_off`` ..) of ``proj`` are rotated on their first ``rot_dims`` entries (entry i with
    i + rot_dims / 2, angle position * freq[i]); k is then multiplied by D^-1/2.  ``v`` [T, H Dv] (a column slice of
    ``proj`` is fine), ``state`` fp32 [slots, H, D, Dv] (read unless the item starts at position 0, written back).
    Returns o fp32 [T, H Dv]."""
    if out is None:
        out = torch.empty(proj.shape[0], H * state.shape[3], dtype=torch.float32, device=proj.device)
    kernels().retention(proj, int(k_off), v, freq, float(mult), int(rot_dims), decay, state, items.cu, items.slots,
                        items.positions, out, int(H))
    return out


def glu(gu: torch.Tensor, out: Optional[torch.Tensor] = None, mode: str = "silu", alpha: float = 1.0,
        limit: float = 0.0) -> torch.Tensor:
    """Gated unit over fused rows [gate | up]: ``silu``: silu(g) * u; ``clamped``: g' = min(g, limit), u' = clamp(u,
    +-limit), g' * sigmoid(alpha g') * (u' + 1)."""
    if out is None:
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
    kernels().glu(gu, out, 0 if mode == "silu" else 1, float(alpha), float(limit))
    return out


# ------------------------------------------------------------------ rotary attention layers, channel-wise decays
def gelu(z: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """z / 2 (1 + erf(z / sqrt 2)); ``z`` and ``out`` may be column slices of row-dense buffers."""
    if out is None:
        out = torch.empty(z.shape[0], z.shape[1], dtype=z.dtype, device=z.device)
    kernels().gelu(z, out)
    return out


def rot_kv_write(src: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 H: int, G: int, scale: float, rot_dims: int = 0, freq: Optional[torch.Tensor] = None, mult: float = 1.0,
                 vfreq: Optional[torch.Tensor] = None, wq: Optional[torch.Tensor] = None, wk: Optional[torch.Tensor] = None,
                 eps: float = 0.0, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Cache side of a rotary attention layer.  ``src`` rows = [q (H D) | k (G D) | v (G Dv)].  With ``wq`` / ``wk`` (fp32
    [D]) q / k are first RMS-normed per head (x / rms(x) * w).  The first ``rot_dims`` entries of every q and k head are
    rotated by the position: entry i < rot_dims / 2 pairs with i + rot_dims / 2, angle position * freq[i], cos and sin
    times ``mult``.  q times ``scale`` -> fp32 [T, H D] (returned); k -> the paged K cache at ``slots`` (-1: no write);
    v -> the paged V cache, with ``vfreq`` (fp32 [Dv / 2]) rotated the same way over all its Dv entries."""
    D = k_cache.shape[2] // G
    if q_out is None:
        q_out = torch.empty(src.shape[0], H * D, dtype=torch.float32, device=src.device)
    kernels().rot_kv_write(src, wq, wk, freq, float(mult), int(rot_dims), vfreq, positions, slots, q_out, k_cache, v_cache,
                           int(H), int(G), float(eps), float(scale))
    return q_out


def head_gate_unrotate(o: torch.Tensor, out: torch.Tensor, positions: torch.Tensor, H: int, gate: Optional[torch.Tensor] = None,
                       vfreq: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t, h] = rot(o[t, h], -position) * sigmoid(gate[t, h]) * scale: the output of an attention over rotated values
    turned back by the row's own position (``vfreq`` None: no rotation), one gate logit per head (``gate`` [T, H])."""
    kernels().head_gate_unrotate(o, gate, vfreq, positions, out, int(H), float(scale))
    return out


def add_rmsnorm(x: torch.Tensor, y: Optional[torch.Tensor], w: torch.Tensor, eps: float, dtype,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (fp32) += y in place (``y`` None: x as it is), and x / rms(x) * w of the new x -> ``dtype`` rows."""
    if out is None:
        out = torch.empty(x.shape[0], x.shape[1], dtype=dtype, device=x.device)
    kernels().add_rmsnorm(x, y, w, out, float(eps))
    return out


def channel_decay_rule(src: torch.Tensor, z: torch.Tensor, state: torch.Tensor, items: StepItems, H: int, G: int,
                       zb: Optional[torch.Tensor] = None, A_log: Optional[torch.Tensor] = None, tau: float = 1.0,
                       beta: Optional[torch.Tensor] = None, unit: bool = False, delta: bool = False,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Linear-attention recurrence with one decay per head and key channel over a step's items.  ``src`` rows
    [q (G D) | k (G D) | v (H Dv)] (head h reads q / k head h // (H / G)); q times D^-1/2, with ``unit`` q and k first
    made unit vectors per head.  Decays g [T, H D] from the logits ``z`` (+ ``zb``): with ``A_log`` (fp32 [H])
    g = exp(-exp(A_log_h) softplus(z)), else g = sigmoid(z)^(1/tau).  Per head, g scaling the rows of S:
    ``delta``: S <- g S; u = sigmoid(beta_h) (v - S^T k); S <- S + k u^T; else S <- g S + k v^T.  o = S^T q.
    ``state`` fp32 [slots, H, D, Dv] (read unless the item starts at position 0, written back).  Returns o fp32
    [T, H Dv]; an fp32 ``src`` is rewritten in place with the q and k that enter the recurrence."""
    T = src.shape[0]
    if out is None:
        out = torch.empty(T, H * state.shape[3], dtype=torch.float32, device=src.device)
    qkv = src if src.dtype == torch.float32 else torch.empty(T, src.shape[1], dtype=torch.float32, device=src.device)
    kernels().chan_rule(src, qkv, z, zb, A_log, 1.0 / float(tau), beta, state, items.cu, items.slots, items.positions, out,
                        int(H), int(G), bool(unit), bool(delta))
    return out
