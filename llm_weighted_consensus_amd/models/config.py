"""Model architecture configs (public shapes, random-init or safetensors weights).

Shapes come from the public model configs (not from the reference, which
runs no model): Llama-3-8B, Mixtral-8x7B, Mistral-7B/e5-mistral-7b and the bge-* BERT encoders.
Small variants exist for tests.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, replace
from pathlib import Path
from typing import Optional, Tuple


@dataclass(frozen=True)
class DecoderConfig:
    name: str
    vocab_size: int
    hidden: int
    layers: int
    heads: int
    kv_heads: int
    head_dim: int
    ffn: int
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_position: int = 8192
    # llama-3 style rope scaling (factor, low_freq_factor, high_freq_factor, original_max_position)
    rope_scaling: Optional[tuple] = None
    # mixture of experts (Mixtral): experts per layer and experts per token; 0 = dense
    num_experts: int = 0
    experts_per_token: int = 0
    tie_embeddings: bool = False
    bos_token_id: int = 1
    eos_token_id: int = 2

    @property
    def qkv_dim(self) -> int:
        return (self.heads + 2 * self.kv_heads) * self.head_dim

    def params(self) -> int:
        d, f = self.hidden, self.ffn
        attn = d * self.qkv_dim + self.heads * self.head_dim * d
        mlp = 3 * d * f * max(1, self.num_experts) + (d * self.num_experts if self.num_experts else 0)
        emb = self.vocab_size * d * (1 if self.tie_embeddings else 2)
        return self.layers * (attn + mlp + 2 * d) + emb + d


@dataclass(frozen=True)
class EncoderConfig:
    name: str
    vocab_size: int
    hidden: int
    layers: int
    heads: int
    ffn: int
    max_position: int = 512
    type_vocab: int = 2
    ln_eps: float = 1e-12
    pooling: str = "cls"  # cls | mean | last

    @property
    def head_dim(self) -> int:
        return self.hidden // self.heads


DECODERS = {
    "llama-3-8b": DecoderConfig("llama-3-8b", 128256, 4096, 32, 32, 8, 128, 14336, rope_theta=500000.0,
                                rms_eps=1e-5, max_position=8192, rope_scaling=(8.0, 1.0, 4.0, 8192),
                                bos_token_id=128000, eos_token_id=128001),
    "mistral-7b": DecoderConfig("mistral-7b", 32000, 4096, 32, 32, 8, 128, 14336, rope_theta=10000.0, rms_eps=1e-5,
                                max_position=32768),
    "mixtral-8x7b": DecoderConfig("mixtral-8x7b", 32000, 4096, 32, 32, 8, 128, 14336, rope_theta=1e6, rms_eps=1e-5,
                                  max_position=32768, num_experts=8, experts_per_token=2),
    # e5-mistral-7b-instruct: Mistral-7B decoder used as an embedder (last-token pooling, 4096-d)
    "e5-mistral-7b": DecoderConfig("e5-mistral-7b", 32000, 4096, 32, 32, 8, 128, 14336, rope_theta=10000.0,
                                   rms_eps=1e-5, max_position=32768),
    # tests / smoke: same code paths, tiny sizes
    "llama-tiny": DecoderConfig("llama-tiny", 4096, 512, 2, 8, 2, 128, 1024, rope_theta=500000.0, max_position=2048,
                                bos_token_id=1, eos_token_id=2),
    "mixtral-tiny": DecoderConfig("mixtral-tiny", 4096, 512, 2, 8, 2, 128, 512, rope_theta=1e6, max_position=2048,
                                  num_experts=4, experts_per_token=2),
}

ENCODERS = {
    "bge-small-en-v1.5": EncoderConfig("bge-small-en-v1.5", 30522, 384, 12, 12, 1536),
    "bge-base-en-v1.5": EncoderConfig("bge-base-en-v1.5", 30522, 768, 12, 12, 3072),
    "bge-large-en-v1.5": EncoderConfig("bge-large-en-v1.5", 30522, 1024, 24, 16, 4096),
    "bert-tiny": EncoderConfig("bert-tiny", 30522, 256, 2, 4, 1024),
}


def decoder_config(name: str, **overrides) -> DecoderConfig:
    cfg = DECODERS[name]
    return replace(cfg, **overrides) if overrides else cfg


def encoder_config(name: str, **overrides) -> EncoderConfig:
    key = name.split("/")[-1].lower()
    if key.startswith("bge-") and not key.endswith("-v1.5") and key + "-en-v1.5" in ENCODERS:
        key = key + "-en-v1.5"
    cfg = ENCODERS[key]
    return replace(cfg, **overrides) if overrides else cfg


# ---------------------------------------------------------------------------------------------
# layer-list decoders: every layer names its own mixer and feed-forward (read from a model folder's config.json)


@dataclass(frozen=True)
class WindowAttentionSpec:
    """A sliding-window attention mixer: H query heads over G key/value heads, key size ``dim`` and value size
    ``vdim`` per head, a window of ``window`` positions (itself and window - 1 before it), the softmax ``scale``
    and whether the layer takes part in the value blending across layers."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    scale: float
    v_mix: bool = False

    @property
    def nq(self) -> int:
        return self.heads * self.dim

    @property
    def nk(self) -> int:
        return self.kv_heads * self.dim

    @property
    def nv(self) -> int:
        return self.kv_heads * self.vdim


@dataclass(frozen=True)
class LayerSpec:
    type: str                      # the mixer's kind ("attention")
    mixer: WindowAttentionSpec
    mlp_kind: Optional[str]        # "dense" or None (no feed-forward in this layer)
    ff: int = 0


@dataclass(frozen=True)
class MadipelConfig:
    """Madipel: parallel layers (one LayerNorm feeds the mixer and the feed-forward, x += m (mixer + ff)) over an
    fp32 residual stream, sinusoidal positions added to the embedding, windowed attention with whole-projection
    q/k RMS norms, per-head temperature and a logarithmic distance bias, xIELU feed-forwards, LayerNorm + scaled
    logits at the output."""
    name: str
    vocab_size: int
    hidden: int
    layer_specs: Tuple[LayerSpec, ...]
    norm_eps: float
    residual_mult: float
    logit_scale: float
    bos_token_id: int = 1
    eos_token_id: int = 2
    sinpos_base: float = 10000.0   # fixed by the design

    architecture = "Madipel"

    # what the engine reads of a decoder config
    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    @property
    def heads(self) -> int:
        return max(L.mixer.heads for L in self.layer_specs)

    @property
    def kv_heads(self) -> int:
        return max(L.mixer.kv_heads for L in self.layer_specs)

    @property
    def head_dim(self) -> int:
        return max(L.mixer.dim for L in self.layer_specs)

    num_experts = 0

    @classmethod
    def from_dict(cls, c: dict, name: str = "madipel") -> "MadipelConfig":
        specs = []
        for L in c["layers"]:
            if L["type"] != "attention":
                raise ValueError(f"Madipel: unknown mixer type {L['type']!r}")
            m = L["mixer"]
            mixer = WindowAttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                        vdim=int(m["vdim"]), window=int(m["mask"]["size"]), scale=float(m["scale"]),
                                        v_mix=bool(m.get("v_mix", False)))
            if mixer.heads % mixer.kv_heads:
                raise ValueError("Madipel: heads must be a multiple of kv_heads")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"Madipel: unknown feed-forward kind {mlp.get('kind')!r}")
            specs.append(LayerSpec(L["type"], mixer, None if mlp is None else "dense", 0 if mlp is None else int(mlp["ff"])))
        return cls(name=name, vocab_size=int(c["vocab"]), hidden=int(c["width"]), layer_specs=tuple(specs),
                   norm_eps=float(c["norm"]["eps"]), residual_mult=float(c["residual_mult"]),
                   logit_scale=float(c["logit_scale"]))

    def params(self) -> int:
        d = self.hidden
        n = 2 * self.vocab_size * d + 2 * d
        for L in self.layer_specs:
            m = L.mixer
            n += 2 * d + d * (m.nq + m.nk + m.nv) + m.nq + m.nk + 1 + 3 * m.heads + d * m.heads * m.vdim
            n += 2 * d * L.ff + (2 if L.mlp_kind else 0)
        return n



# ------------------------------------------------------------------ Merudra
@dataclass(frozen=True)
class GatedAttentionSpec:
    """Causal softmax attention without rotation: per-head unit-RMS q and k, the keys as projected are the values,
    a query temperature that grows with the logarithm of the position, a sigmoid output gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float
    temp_every: int

    @property
    def nq(self) -> int:
        return self.heads * self.dim

    @property
    def nk(self) -> int:
        return self.kv_heads * self.dim

    @property
    def nv(self) -> int:
        return self.kv_heads * self.vdim


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta rule: q, k over ``kv_heads`` heads of size ``dim``, v over ``heads`` heads of size ``vdim``,
    each behind a short causal convolution with ``conv`` taps."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @property
    def nq(self) -> int:
        return self.kv_heads * self.dim

    @property
    def nv(self) -> int:
        return self.heads * self.vdim


@dataclass(frozen=True)
class RoutedExpertsSpec:
    experts: int       # real experts (each a gated feed-forward of inner width ff)
    identity: int      # further router outputs whose expert is the identity
    top: int
    ff: int


@dataclass(frozen=True)
class MerudraLayerSpec:
    type: str                                   # "attention" | "delta"
    mixer: object                               # GatedAttentionSpec | DeltaRuleSpec
    mlp: Optional[RoutedExpertsSpec]            # None: no feed-forward in this layer


@dataclass(frozen=True)
class MerudraConfig:
    """Merudra: an fp32 residual stream; every sublayer reads x + causal_conv(x), its result is gated by
    sigmoid(W x + b), RMS-normalised and added; mixers are gated causal attention or gated delta rule layers;
    feed-forwards are routed experts with identity experts; a per-layer token embedding is added after the
    feed-forward; the next layer reads a learned average of all earlier layers' results."""
    name: str
    vocab_size: int
    hidden: int
    layer_specs: Tuple[MerudraLayerSpec, ...]
    norm_eps: float
    canon_taps: int
    side_dim: int
    bos_token_id: int = 1
    eos_token_id: int = 2

    architecture = "Merudra"
    num_experts = 0   # the engine's expert-parallel planning does not apply

    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    @property
    def attention_layers(self) -> Tuple[int, ...]:
        return tuple(i for i, L in enumerate(self.layer_specs) if L.type == "attention")

    @property
    def heads(self) -> int:
        return max(L.mixer.heads for L in self.layer_specs)

    @property
    def kv_heads(self) -> int:
        return max(L.mixer.kv_heads for L in self.layer_specs)

    @property
    def head_dim(self) -> int:
        return max(L.mixer.dim for L in self.layer_specs)

    @classmethod
    def from_dict(cls, c: dict, name: str = "merudra") -> "MerudraConfig":
        specs = []
        for L in c["layers"]:
            m = L["mixer"]
            if L["type"] == "attention":
                t = m.get("q_temp") or {}
                mixer = GatedAttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                           vdim=int(m["vdim"]), scale=float(m["scale"]),
                                           temp_coef=float(t.get("coef", 0.0)), temp_every=int(t.get("every", 0)))
                if mixer.vdim != mixer.dim:
                    raise ValueError("Merudra: the values are the keys, so vdim must equal dim")
            elif L["type"] == "delta":
                mixer = DeltaRuleSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                      vdim=int(m["vdim"]), conv=int(m["conv"]))
            else:
                raise ValueError(f"Merudra: unknown mixer type {L['type']!r}")
            if mixer.heads % mixer.kv_heads:
                raise ValueError("Merudra: heads must be a multiple of kv_heads")
            mlp = L.get("mlp")
            spec = None
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ValueError(f"Merudra: unknown feed-forward kind {mlp.get('kind')!r}")
                r = mlp["router"]
                spec = RoutedExpertsSpec(experts=int(r["experts"]), identity=int(r.get("identity", 0)), top=int(r["top"]),
                                         ff=int(mlp["expert"]["ff"]))
                if not 1 <= spec.top <= spec.experts + spec.identity:
                    raise ValueError("Merudra: router.top out of range")
            specs.append(MerudraLayerSpec(L["type"], mixer, spec))
        return cls(name=name, vocab_size=int(c["vocab"]), hidden=int(c["width"]), layer_specs=tuple(specs),
                   norm_eps=float(c["norm"]["eps"]), canon_taps=int(c["canon"]["taps"]),
                   side_dim=int(c["token_side"]["dim"]))

    def params(self) -> int:
        d = self.hidden
        n = 2 * self.vocab_size * d + d + self.vocab_size * self.side_dim * self.layers
        for i, L in enumerate(self.layer_specs):
            m = L.mixer
            n += d + d * self.canon_taps + (d * d + d) + (i + 2) + 2 * d * self.side_dim + d
            if L.type == "attention":
                n += d * (2 * m.nq + m.nk) + m.nq + m.nk + d * m.heads * m.vdim
            else:
                n += d * (2 * m.nq + 2 * m.nv + 2 * m.heads) + (2 * m.nq + m.nv) * m.conv + 2 * m.heads + m.vdim + d * m.nv
            if L.mlp is not None:
                e = L.mlp
                n += d + d * self.canon_taps + (d * d + d)
                n += e.experts * 3 * d * e.ff + (e.experts + e.identity) * (d + 1)
        return n


# ------------------------------------------------------------------ Limatar
@dataclass(frozen=True)
class RotarySpec:
    """Rotation by position of the first ``dims`` entries of a head: pair i turns by position * f_i, f_i =
    base^(-2i/dims).  ``scaling`` (factor, original, fast, slow) stretches the slow pairs (frequency blending over a
    ramp of the pair index) and multiplies the cos / sin tables by 0.1 ln(factor) + 1."""
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None   # factor, original, fast, slow

    def scaling_dict(self) -> Optional[dict]:
        if self.scaling is None:
            return None
        f, o, a, b = self.scaling
        return {"factor": f, "original": o, "fast": a, "slow": b}

    @classmethod
    def from_dict(cls, r: dict) -> "RotarySpec":
        sc = r.get("scaling")
        return cls(dims=int(r["dims"]), base=float(r["base"]),
                   scaling=None if not sc else (float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                                float(sc["slow"])))


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal softmax attention whose queries and keys / values pass through low-rank latents (``q_rank``,
    ``kv_rank``); per head ``dim`` unrotated and ``rot_dim`` rotated query / key entries (the rotated key part is one
    vector for all heads, pairs interleaved), values of ``vdim``; a learned sink per head in the softmax's
    denominator; a sigmoid output gate."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: RotarySpec

    kv_heads = 1   # one cached row (latent + rotated part) serves every head

    @property
    def nq(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def nv(self) -> int:
        return self.heads * self.vdim


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head: S <- a_h S + k v^T, o = S^T q; q, k rotated ("rotate half"
    pairing), per-head unit RMS on o, a silu gate."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: RotarySpec

    kv_heads = 0

    @property
    def nq(self) -> int:
        return self.heads * self.dim

    @property
    def nv(self) -> int:
        return self.heads * self.vdim


@dataclass(frozen=True)
class ClampedGluSpec:
    """Dense feed-forward W_down (g' sigmoid(alpha g') (u' + 1)) with g' = min(g, limit), u' = clamp(u, +-limit)."""
    ff: int
    limit: float
    alpha: float = 1.702   # fixed by the design


@dataclass(frozen=True)
class TopkExpertsSpec:
    """Routed experts (silu-gated, no biases): the ``top`` largest router logits (+ bias) choose, the weights are the
    softmax over the chosen logits; ``shared_ff`` > 0: one more expert of that width runs for every token."""
    experts: int
    top: int
    ff: int
    shared_ff: int


@dataclass(frozen=True)
class LimatarLayerSpec:
    type: str                 # "latent_attention" | "retention"
    mixer: object             # LatentAttentionSpec | RetentionSpec
    mlp: object               # ClampedGluSpec | TopkExpertsSpec | None


@dataclass(frozen=True)
class LimatarConfig:
    """Limatar: an fp32 residual stream with a norm before AND after every sublayer (weights stored around zero),
    mixers = low-rank attention with sinks or retention, feed-forwards = a clamped gated unit or routed experts with a
    shared expert, a span of layers that runs several times in a row with the same weights (every pass has its own
    cache and state), output weights tied to the embedding."""
    name: str
    vocab_size: int
    hidden: int
    layer_specs: Tuple[LimatarLayerSpec, ...]
    norm_eps: float
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    bos_token_id: int = 1
    eos_token_id: int = 2

    architecture = "Limatar"
    num_experts = 0   # the engine's expert-parallel planning does not apply

    @property
    def runs(self) -> Tuple[int, ...]:
        """The layer index of every layer run, in execution order (the looped span repeated in a row)."""
        n = len(self.layer_specs)
        a, b = self.loop_start, self.loop_stop
        return tuple(range(a)) + tuple(range(a, b)) * self.loop_times + tuple(range(b, n))

    @property
    def layers(self) -> int:
        return len(self.runs)

    @property
    def heads(self) -> int:
        return max(L.mixer.heads for L in self.layer_specs)

    @property
    def kv_heads(self) -> int:
        return 1

    @property
    def head_dim(self) -> int:
        return max(L.mixer.dim for L in self.layer_specs)

    @classmethod
    def from_dict(cls, c: dict, name: str = "limatar") -> "LimatarConfig":
        specs = []
        for L in c["layers"]:
            m = L["mixer"]
            if L["type"] == "latent_attention":
                rot = RotarySpec.from_dict(m["rot"])
                mixer = LatentAttentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                                            vdim=int(m["vdim"]), q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]),
                                            scale=float(m["scale"]), rot=rot)
                if rot.dims != mixer.rot_dim or rot.dims % 2:
                    raise ValueError("Limatar: a latent attention layer rotates its whole rot_dim part (an even size)")
            elif L["type"] == "retention":
                rot = RotarySpec.from_dict(m["rot"])
                mixer = RetentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                      decay=tuple(float(a) for a in m["decay"]), rot=rot)
                if len(mixer.decay) != mixer.heads:
                    raise ValueError("Limatar: one decay per retention head")
                if rot.dims % 2 or rot.dims > mixer.dim:
                    raise ValueError("Limatar: rot.dims must be even and at most dim")
            else:
                raise ValueError(f"Limatar: unknown mixer type {L['type']!r}")
            mlp = L.get("mlp")
            spec = None
            if mlp is not None:
                if mlp.get("kind") == "dense":
                    spec = ClampedGluSpec(ff=int(mlp["ff"]), limit=float(mlp["limit"]))
                elif mlp.get("kind") == "moe":
                    r = mlp["router"]
                    sh = mlp.get("shared")
                    spec = TopkExpertsSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                                           shared_ff=int(sh["ff"]) if sh else 0)
                    if not 1 <= spec.top <= spec.experts:
                        raise ValueError("Limatar: router.top out of range")
                else:
                    raise ValueError(f"Limatar: unknown feed-forward kind {mlp.get('kind')!r}")
            specs.append(LimatarLayerSpec(L["type"], mixer, spec))
        lp = c.get("loop") or {}
        a, b, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
        if not (0 <= a <= b <= len(specs)) or times < 1:
            raise ValueError("Limatar: loop span out of range")
        return cls(name=name, vocab_size=int(c["vocab"]), hidden=int(c["width"]), layer_specs=tuple(specs),
                   norm_eps=float(c["norm"]["eps"]), loop_start=a, loop_stop=b, loop_times=times)

    def params(self) -> int:
        d = self.hidden
        n = self.vocab_size * d + 2 * d
        for L in self.layer_specs:
            m = L.mixer
            n += 2 * d
            if L.type == "latent_attention":
                n += d * (m.q_rank + m.kv_rank + m.rot_dim + m.nv) + m.q_rank + m.kv_rank + m.q_rank * m.nq
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads + d * m.nv
            else:
                n += d * (2 * m.nq + 2 * m.nv) + d * m.nv
            if isinstance(L.mlp, ClampedGluSpec):
                n += 2 * d + 3 * d * L.mlp.ff
            elif L.mlp is not None:
                n += 2 * d + (L.mlp.experts * L.mlp.ff + L.mlp.shared_ff) * 3 * d + L.mlp.experts * (d + 1)
        return n


# ------------------------------------------------------------------ Rerozen
@dataclass(frozen=True)
class RotaryAttentionSpec:
    """Causal softmax attention with rotary positions on the first ``rot.dims`` entries of every q / k head (rotate-half
    pairing), GQA, a sigmoid gate per head on the output.  ``chunk``: positions are cut into chunks of that many from
    position 0 and a row sees only its own chunk.  Options: biases on q / k / v; a per-head RMS norm of q and k with one
    weight for all heads (before the rotation); a short causal convolution (``conv`` taps, 0 = none) behind the three
    projections; values rotated by their own position over all ``vdim`` entries (plain frequencies of ``rot.base``) and
    the head's output turned back by the query's position; ``sink``: one added to the softmax's denominator."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int
    rot: RotarySpec
    bias: bool = False
    qk_norm: bool = False
    conv: int = 0
    rotate_values: bool = False
    sink: bool = False

    @property
    def nq(self) -> int:
        return self.heads * self.dim

    @property
    def nk(self) -> int:
        return self.kv_heads * self.dim

    @property
    def nv(self) -> int:
        return self.kv_heads * self.vdim


@dataclass(frozen=True)
class ChannelDecaySpec:
    """A linear-attention mixer whose state rows decay per head AND key channel; the decay logits come through a low-rank
    pair of projections (``a_rank``; 0: read from the checkpoint's tensor shapes).
    ``kind`` "gla": S <- diag(alpha) S + k v^T with alpha = sigmoid(z)^(1/tau), q times dim^-1/2, silu gate, ``kv_heads``
    = ``heads``.  ``kind`` "delta": the gated delta rule with unit q / k behind a short convolution (``conv`` taps) + silu,
    q / k over ``kv_heads`` heads, decays exp(-exp(A_log) softplus(z + dt_bias)), a low-rank sigmoid gate (``g_rank``)."""
    kind: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    tau: float = 1.0
    conv: int = 0
    a_rank: int = 0
    g_rank: int = 0

    @property
    def nq(self) -> int:
        return self.kv_heads * self.dim

    @property
    def nv(self) -> int:
        return self.heads * self.vdim

    @property
    def nd(self) -> int:
        return self.heads * self.dim


@dataclass(frozen=True)
class RerozenLayerSpec:
    type: str                       # "parallel" (attention beside gated linear attention) | "parallel_2" (... delta rule)
    left: RotaryAttentionSpec
    right: ChannelDecaySpec
    left_scale: float
    right_scale: float
    ff: int                         # 0: no feed-forward in this layer

    @property
    def mixer(self) -> RotaryAttentionSpec:
        return self.left


@dataclass(frozen=True)
class RerozenConfig:
    """Rerozen: a pre-norm fp32 residual stream; every sublayer reads h + causal_conv(h) of its normed input; a mixer is
    TWO mixers side by side on the same input, a chunked rotary attention and a channel-decay linear attention, their
    results added with fixed scales; ungated gelu feed-forwards; scaled embedding and logits."""
    name: str
    vocab_size: int
    hidden: int
    layer_specs: Tuple[RerozenLayerSpec, ...]
    norm_eps: float
    canon_taps: int
    embed_scale: float
    logit_scale: float
    bos_token_id: int = 1
    eos_token_id: int = 2

    architecture = "Rerozen"
    num_experts = 0   # the engine's expert-parallel planning does not apply

    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    @property
    def heads(self) -> int:
        return max(L.left.heads for L in self.layer_specs)

    @property
    def kv_heads(self) -> int:
        return max(L.left.kv_heads for L in self.layer_specs)

    @property
    def head_dim(self) -> int:
        return max(L.left.dim for L in self.layer_specs)

    @classmethod
    def from_dict(cls, c: dict, name: str = "rerozen") -> "RerozenConfig":
        specs = []
        for L in c["layers"]:
            if L["type"] not in ("parallel", "parallel_2"):
                raise ValueError(f"Rerozen: unknown mixer type {L['type']!r}")
            two = L["type"] == "parallel_2"
            m = L["mixer"]
            a, b = m["left"], m["right"]
            rot = RotarySpec.from_dict(a["rot"])
            left = RotaryAttentionSpec(heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                                       scale=float(a["scale"]), chunk=int(a["mask"]["size"]), rot=rot, bias=not two,
                                       qk_norm=not two, conv=int(a["conv"]) if two else 0, rotate_values=two, sink=two)
            if left.heads % left.kv_heads:
                raise ValueError("Rerozen: heads must be a multiple of kv_heads")
            if rot.dims % 2 or rot.dims > left.dim or left.chunk < 1 or (two and (left.vdim % 2 or left.conv < 1)):
                raise ValueError("Rerozen: rot.dims even and at most dim, mask.size >= 1, rotated values of even size")
            if two:
                right = ChannelDecaySpec("delta", heads=int(b["heads"]), kv_heads=int(b["kv_heads"]), dim=int(b["dim"]),
                                         vdim=int(b["vdim"]), conv=int(b["conv"]), a_rank=int(b.get("a_rank", 0)),
                                         g_rank=int(b.get("g_rank", 0)))
                if right.conv < 1:
                    raise ValueError("Rerozen: conv taps must be at least 1")
            else:
                right = ChannelDecaySpec("gla", heads=int(b["heads"]), kv_heads=int(b["heads"]), dim=int(b["dim"]),
                                         vdim=int(b["vdim"]), tau=float(b["tau"]), a_rank=int(b.get("a_rank", 0)))
            if right.heads % right.kv_heads:
                raise ValueError("Rerozen: heads must be a multiple of kv_heads")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"Rerozen: unknown feed-forward kind {mlp.get('kind')!r}")
            specs.append(RerozenLayerSpec(L["type"], left, right, float(m["left_scale"]), float(m["right_scale"]),
                                          0 if mlp is None else int(mlp["ff"])))
        return cls(name=name, vocab_size=int(c["vocab"]), hidden=int(c["width"]), layer_specs=tuple(specs),
                   norm_eps=float(c["norm"]["eps"]), canon_taps=int(c["canon"]["taps"]),
                   embed_scale=float(c["embedding"]["scale"]), logit_scale=float(c["logit_scale"]))

    def with_ranks(self, shapes: dict) -> "RerozenConfig":
        """The config with every low-rank width that it leaves open taken from a checkpoint's tensor shapes."""
        specs = []
        for i, L in enumerate(self.layer_specs):
            r, p = L.right, f"l{i}.mix.right."
            ar = r.a_rank or int(shapes[p + "a1"][0])
            gr = r.g_rank or (int(shapes[p + "g1"][0]) if r.kind == "delta" else 0)
            specs.append(replace(L, right=replace(r, a_rank=ar, g_rank=gr)))
        return replace(self, layer_specs=tuple(specs))

    def params(self) -> int:
        d = self.hidden
        n = 2 * self.vocab_size * d + d
        for L in self.layer_specs:
            a, r = L.left, L.right
            n += d + d * self.canon_taps + d * (a.nq + a.nk + a.nv + a.heads) + d * a.heads * a.vdim
            n += (a.nq + a.nk + a.nv) * (a.conv + (1 if a.bias else 0)) + (2 * a.dim if a.qk_norm else 0)
            n += d * (2 * r.nq + r.nv) + d * r.nv + r.vdim + d * r.a_rank + r.a_rank * r.nd + r.nd
            if r.kind == "delta":
                n += (2 * r.nq + r.nv) * r.conv + d * r.heads + r.heads + d * r.g_rank + r.g_rank * r.nv
            else:
                n += d * r.nv
            if L.ff:
                n += d + d * self.canon_taps + 2 * d * L.ff
        return n


# config.json "architecture" -> config class of the layer-list decoders
ARCHITECTURES = {"Madipel": MadipelConfig, "Merudra": MerudraConfig, "Limatar": LimatarConfig, "Rerozen": RerozenConfig}


def load_model_config(model_dir) -> object:
    """The config object of a model folder (config.json with an "architecture" this framework knows)."""
    path = Path(model_dir) / "config.json"
    with open(path) as f:
        c = json.load(f)
    arch = c.get("architecture")
    if arch not in ARCHITECTURES:
        raise ValueError(f"{path}: unknown architecture {arch!r} (known: {sorted(ARCHITECTURES)})")
    return ARCHITECTURES[arch].from_dict(c, name=Path(model_dir).name or arch.lower())
