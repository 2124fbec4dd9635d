"""Limatar decoder on the fp32-residual kernel set (``ops/res32.py``, ``csrc/kernels/res32``).

The residual stream x is fp32; every norm is x / rms(x) * (1 + w) (the stored weights are offsets from one, the sum
is formed once at load).  A layer run over the T rows of a step (decode rows and prompt-portion rows alike):

    h      = norm1(x)                                   res32.rmsnorm_rows
    low-rank attention layer:
      proj = h @ [Wdq | Wdkv | Wg]^T                     ONE GEMM
      cq   = rms_norm(proj_dq) * w;  cache <- [rms_norm(c) * w | rot(k_r)] and c again as the value row
                                                         res32.latent_kv_write (one cached row serves every head)
      q    = cq @ Wuq^T                                  GEMM
      qf   = [ (q_unrotated Wuk) * scale | rot(q_r) * scale ]   batched GEMM per head + res32.latent_q_rows: the keys'
                                                         up-projection is applied to the query, so scores are taken
                                                         against the cached latent itself
      o_c  = softmax with a sink over the cache          res32.window_attn (G = 1: all heads read the one cached row)
      a    = (o_c Wuv^T per head) * sigmoid(proj_g)      batched GEMM + res32.gate_mul
      (bf16, cached rows wider than the portion kernel takes: prompt portions instead attend per head over keys
       [Wuk c | rotated part] and values Wuv c up-projected from their sequences' cached rows into pages of their own,
       res32.latent_expand_write; decode rows stay on the cached rows)
    retention layer:
      proj = h @ [Wq | Wk | Wv | Wg]^T                   ONE GEMM
      o    = S <- a_h S + k v^T, S^T q over the slot     res32.retention (rotation of q, k inside; state fp32 [H, D, Dv])
      a    = o / rms(o) per head * silu(proj_g)          res32.head_norm_gate
    x     += norm1b(a @ Wo^T);  h2 = norm2(x)            res32.gated_norm_residual (no gate; both norms in one pass)
    dense:   y = (glu_clamped(h2 @ [Wgate | Wup]^T)) @ Wdown^T             res32.glu
    experts: top-k of the router's logits + bias, softmax over the chosen  res32.router (fp32)
             y = sum_j s_j expert_j(h2) + shared(h2)                       res32.expert_rows / grouped GEMMs, moe_combine
    x     += norm2b(y);  h = the next run's norm1(x)     res32.gated_norm_residual

``cfg.runs`` lists the layer of every run: a looped span repeats in a row with the same weights, and every run has its
own pages in the paged cache (attention) or its own matrix in the recurrent-state slots (retention).
Logits = norm(x) @ embed^T (tied).  ``dtype=torch.float32`` runs every GEMM, activation and the cache in true fp32.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Callable, Dict, List, Optional

import numpy as np
import torch
import torch.nn.functional as F

from .. import ops
from ..ops import gemm_plan, res32
from .cache import PagedLayerCache
from .config import ClampedGluSpec, LimatarConfig, TopkExpertsSpec
from .state import RecurrentStatePool

UNBOUNDED = 1 << 30  # "window" of a causal attention without one


def _up(n: int, m: int) -> int:
    return -(-n // m) * m


def _core_size(n: int) -> int:
    """The next head size the matrix-core attention kernels are built for (beyond 128: a multiple of 8)."""
    for c in (32, 64, 128):
        if n <= c:
            return c
    return _up(n, 8)


@dataclass
class StepAttention:
    """How a step's rows reach the paged cache: ``n_dec`` decode rows (row b reads ``dec_tables[b]``), then prompt
    portions described by ``chunk`` (block tables, row offsets, key counts; host copies of the counts in "lens")."""
    n_dec: int
    dec_tables: Optional[torch.Tensor]
    chunk: Optional[dict]
    scratch: Dict[object, object] = field(default_factory=dict)   # per-step data shared by the layer runs


@dataclass
class LimatarLayer:
    norm1: torch.Tensor                  # fp32, 1 + w
    norm1b: torch.Tensor
    norm2: Optional[torch.Tensor]
    norm2b: Optional[torch.Tensor]
    w_in: torch.Tensor                   # fused input-side projections of the mixer
    w_o: torch.Tensor
    extra: Dict[str, torch.Tensor] = field(default_factory=dict)


class LimatarModel:
    paged_prefill = True      # whole prompts run as one portion over the paged cache (engine._run_prefill)
    supports_cascade = False
    graph_safe = True
    float_logits = True
    has_state = True          # the engine gives every sequence a recurrent-state slot

    # experts at least this large (d * ff) go through the grouped matrix-core GEMMs of the full kernel extension
    GROUPED_MIN = 1 << 18

    def __init__(self, cfg: LimatarConfig, device="cuda", dtype=torch.bfloat16, seed: int = 0,
                 weights_path: Optional[str] = None, max_position: Optional[int] = None):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Limatar runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        if self.device.type != "cuda":
            raise RuntimeError("Limatar runs on the GPU kernels only (no CPU path)")
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        K = res32.kernels()
        for L in cfg.layer_specs:
            if L.type == "retention" and L.mixer.dim > K.retention_max_dim():
                raise ValueError("Limatar: retention head size beyond what the kernel is built for")
            if L.type == "latent_attention" and _up(L.mixer.kv_rank, 8) > 512:
                raise ValueError("Limatar: kv_rank beyond what the attention kernels are built for")
            if isinstance(L.mlp, TopkExpertsSpec) and L.mlp.experts > K.router_max_outputs():
                raise ValueError("Limatar: too many router outputs")
        self.logit_width = _up(cfg.vocab_size, 32)
        self.runs = cfg.runs
        # run -> index of its pages' views in the paged cache (attention runs only)
        self.cache_index = {}
        for ri, li in enumerate(self.runs):
            if cfg.layer_specs[li].type == "latent_attention":
                self.cache_index[ri] = len(self.cache_index)
        self._mm32 = self._probe_mm32()
        raw = self._read(weights_path) if weights_path else self._random(seed)
        self._assemble(raw)
        self.g8_ws = None
        self.on_layer: Optional[Callable[[int, torch.Tensor], None]] = None
        self._zeros_h: Dict[int, torch.Tensor] = {}

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self) -> dict:
        """name -> shape of every tensor of a checkpoint of this config."""
        cfg, d = self.cfg, self.cfg.hidden
        out = {"embed": (cfg.vocab_size, d), "embed.norm": (d,), "final.norm": (d,)}
        for i, L in enumerate(cfg.layer_specs):
            m, p = L.mixer, f"l{i}."
            out.update({p + "norm1": (d,), p + "norm1b": (d,)})
            if L.type == "latent_attention":
                out.update({p + "mix.dq": (m.q_rank, d), p + "mix.dq.norm": (m.q_rank,), p + "mix.uq": (m.nq, m.q_rank),
                            p + "mix.dkv": (m.kv_rank + m.rot_dim, d), p + "mix.dkv.norm": (m.kv_rank,),
                            p + "mix.uk": (m.heads * m.dim, m.kv_rank), p + "mix.uv": (m.nv, m.kv_rank),
                            p + "mix.sink": (m.heads,), p + "mix.g": (m.nv, d), p + "mix.o": (d, m.nv)})
            else:
                out.update({p + "mix.q": (m.nq, d), p + "mix.k": (m.nq, d), p + "mix.v": (m.nv, d), p + "mix.g": (m.nv, d),
                            p + "mix.o": (d, m.nv)})
            e = L.mlp
            if e is not None:
                out.update({p + "norm2": (d,), p + "norm2b": (d,)})
            if isinstance(e, ClampedGluSpec):
                out.update({p + "mlp.gate": (e.ff, d), p + "mlp.up": (e.ff, d), p + "mlp.down": (d, e.ff)})
            elif isinstance(e, TopkExpertsSpec):
                out.update({p + "mlp.router": (e.experts, d), p + "mlp.router.b": (e.experts,)})
                for x in range(e.experts):
                    out.update({f"{p}mlp.e{x}.gate": (e.ff, d), f"{p}mlp.e{x}.up": (e.ff, d), f"{p}mlp.e{x}.down": (d, e.ff)})
                if e.shared_ff:
                    out.update({p + "mlp.shared.gate": (e.shared_ff, d), p + "mlp.shared.up": (e.shared_ff, d),
                                p + "mlp.shared.down": (d, e.shared_ff)})
        return out

    def _random(self, seed: int) -> dict:
        """Random weights of the config's shapes (benchmarks, tests): bf16-representable values."""
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        d = self.cfg.hidden
        out = {}
        for name, shape in self.tensor_shapes().items():
            leaf = name.split(".")[-1]
            if leaf in ("norm1", "norm2", "norm1b", "norm2b") or name in ("final.norm", "embed.norm"):
                t = 0.1 * torch.randn(shape, generator=g)            # stored around zero
            elif leaf == "norm":
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)      # the latents' plain weights
            elif leaf == "sink":
                t = torch.randn(shape, generator=g)
            elif leaf == "b":
                t = 0.1 * torch.randn(shape, generator=g)
            elif name == "embed":
                t = torch.randn(shape, generator=g)
            else:
                t = torch.randn(shape, generator=g) / math.sqrt(shape[-1] if len(shape) > 1 else d)
            out[name] = t.to(torch.bfloat16)
        return out

    def _read(self, path: str) -> dict:
        from safetensors.torch import load_file

        p = Path(path)
        files = sorted(p.glob("*.safetensors")) if p.is_dir() else [p]
        if not files:
            raise FileNotFoundError(f"no .safetensors under {path}")
        sd = {}
        for f in files:
            sd.update(load_file(str(f), device="cpu"))
        for name, shape in self.tensor_shapes().items():
            if name not in sd:
                raise KeyError(f"{path}: tensor {name} missing")
            if tuple(sd[name].shape) != tuple(shape):
                raise ValueError(f"{path}: {name} has shape {tuple(sd[name].shape)}, the config says {tuple(shape)}")
        return sd

    def _assemble(self, sd: dict) -> None:
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def t(name):
            return sd[name].to(device=dev, dtype=dt).contiguous()

        def f32(name):
            return sd[name].to(device=dev, dtype=torch.float32).contiguous()

        def one_plus(name):
            return (1.0 + f32(name)).contiguous()

        self.embed = t("embed")
        self.embed_norm, self.final_w = one_plus("embed.norm"), one_plus("final.norm")
        self.layers: List[LimatarLayer] = []
        for i, L in enumerate(cfg.layer_specs):
            m, p = L.mixer, f"l{i}."
            x: Dict[str, torch.Tensor] = {}
            x["freq"], x["rot_mult"] = res32.rope_frequencies(m.rot.dims, m.rot.base, m.rot.scaling_dict(), dev)
            if L.type == "latent_attention":
                w_in = torch.cat([t(p + "mix.dq"), t(p + "mix.dkv"), t(p + "mix.g")], 0).contiguous()
                x["dq_norm"], x["dkv_norm"], x["sink"] = f32(p + "mix.dq.norm"), f32(p + "mix.dkv.norm"), f32(p + "mix.sink")
                x["w_uq"] = t(p + "mix.uq")
                x["w_uk"] = t(p + "mix.uk").view(m.heads, m.dim, m.kv_rank)                               # [H, D, C]
                x["w_uv_t"] = t(p + "mix.uv").view(m.heads, m.vdim, m.kv_rank).transpose(1, 2).contiguous()  # [H, C, Dv]
                if self.expanded_head_sizes(m) is not None:
                    x["w_ukv"] = torch.cat([t(p + "mix.uk"), t(p + "mix.uv")], 0).contiguous()
            else:
                w_in = torch.cat([t(p + "mix.q"), t(p + "mix.k"), t(p + "mix.v"), t(p + "mix.g")], 0).contiguous()
                x["decay"] = torch.tensor(m.decay, dtype=torch.float32, device=dev)
            e = L.mlp
            if isinstance(e, ClampedGluSpec):
                x["w_gu"] = torch.cat([t(p + "mlp.gate"), t(p + "mlp.up")], 0).contiguous()
                x["w_down"] = t(p + "mlp.down")
            elif isinstance(e, TopkExpertsSpec):
                x["router"], x["router_b"] = f32(p + "mlp.router"), f32(p + "mlp.router.b")
                if self._mm32 and bool((x["router"].to(dt).float() == x["router"]).all()):
                    x["router_t"] = x["router"].to(dt).t().contiguous()
                x["w_gu"] = torch.stack([torch.cat([t(f"{p}mlp.e{j}.gate"), t(f"{p}mlp.e{j}.up")], 0)
                                         for j in range(e.experts)]).contiguous()
                x["w_down"] = torch.stack([t(f"{p}mlp.e{j}.down") for j in range(e.experts)]).contiguous()
                if e.shared_ff:
                    x["ws_gu"] = torch.cat([t(p + "mlp.shared.gate"), t(p + "mlp.shared.up")], 0).contiguous()
                    x["ws_down"] = t(p + "mlp.shared.down")
            has = e is not None
            self.layers.append(LimatarLayer(norm1=one_plus(p + "norm1"), norm1b=one_plus(p + "norm1b"),
                                            norm2=one_plus(p + "norm2") if has else None,
                                            norm2b=one_plus(p + "norm2b") if has else None, w_in=w_in, w_o=t(p + "mix.o"),
                                            extra=x))

    # ------------------------------------------------------------------ GEMMs
    def _probe_mm32(self) -> bool:
        """Whether this torch build multiplies bf16 matrices into an fp32 result (router logits, absorbed queries)."""
        if self.dtype != torch.bfloat16:
            return False
        try:
            a = torch.zeros(2, 8, 16, dtype=self.dtype, device=self.device)
            return (torch.mm(a[0], a[0].t(), out_dtype=torch.float32).dtype == torch.float32
                    and torch.bmm(a, a.transpose(1, 2), out_dtype=torch.float32).dtype == torch.float32)
        except (TypeError, RuntimeError):
            return False

    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        if self.g8_ws is not None:
            return gemm_plan.linear(x, w, ws=self.g8_ws)
        return F.linear(x, w)

    def tune_gemms(self, M: int, bucket: bool = False, lm_head: bool = True, only=None) -> None:
        """Pick the backend of the projections at M rows by timing the library and the hand-written cores (the engine
        calls this before it captures a decode bucket's graph).  bf16 only, and only where the full kernel extension is
        built; otherwise every GEMM stays on the library."""
        if self.dtype != torch.bfloat16 or only is not None or not ops.available():
            return
        if self.g8_ws is None:
            self.g8_ws = ops.new_gemm8p_workspace(self.device)
        seen = set()
        ws = [w for L in self.layers for w in (L.w_in, L.w_o, L.extra.get("w_uq"), L.extra.get("ws_gu"), L.extra.get("ws_down"))]
        ws += [L.extra[k] for L in self.layers for k in ("w_gu", "w_down") if k in L.extra and L.extra[k].dim() == 2]
        for w in ws + ([self.embed] if lm_head else []):
            if w is not None and tuple(w.shape) not in seen and w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0:
                seen.add(tuple(w.shape))
                gemm_plan.tune(torch.randn(M, w.shape[1], device=self.device).to(self.dtype), w, ws=self.g8_ws, bucket=bucket)

    # ------------------------------------------------------------------ cache and state
    def latent_row_sizes(self, m) -> tuple:
        """(key row, value row) sizes of a low-rank attention layer's cached token: [latent | rotated part] and the
        latent, padded with zeros.  bf16: up to the next size the matrix-core attention kernels are built for (32, 64,
        128; one wide row of 576 / 512 for latents above 288 entries), else to a multiple of 8 (16-byte rows)."""
        nk, nv = m.kv_rank + m.rot_dim, m.kv_rank
        if self.dtype == torch.bfloat16:
            if nk <= 128:
                return _core_size(nk), _core_size(nv)
            if 288 < nk <= 576 and nv <= 512:
                return 576, 512
        return _up(nk, 8), _up(nv, 8)

    def expanded_head_sizes(self, m) -> Optional[tuple]:
        """(key, value) sizes per head of the up-projected keys [unrotated | rotated part] and values that prompt
        portions attend over when the cached rows themselves are too wide for the portion kernel; None: not used."""
        K = res32.kernels()
        if self.dtype != torch.bfloat16 or K.window_attn_mfma_ok(*self.latent_row_sizes(m)):
            return None
        dk = _core_size(m.dim + m.rot_dim) if m.dim + m.rot_dim <= 128 else _up(m.dim + m.rot_dim, 64)
        dv = _core_size(m.vdim)
        return (dk, dv) if K.window_attn_mfma_ok(dk, dv) else None

    def _layer_dims(self):
        return [self.latent_row_sizes(self.cfg.layer_specs[self.runs[ri]].mixer) for ri in sorted(self.cache_index)]

    def new_cache(self, num_blocks: int, block_size: int) -> PagedLayerCache:
        return PagedLayerCache(self._layer_dims(), num_blocks, block_size, self.device, self.dtype)

    def bytes_per_block(self, block_size: int) -> int:
        n = PagedLayerCache.elems_per_block(self._layer_dims(), block_size) * (4 if self.dtype == torch.float32 else 2)
        return max(n, 16)

    def state_fields(self):
        """(name, shape) of every per-sequence state tensor: one retention matrix set per retention RUN."""
        out = []
        for ri, li in enumerate(self.runs):
            L = self.cfg.layer_specs[li]
            if L.type == "retention":
                out.append((f"S.{ri}", (L.mixer.heads, L.mixer.dim, L.mixer.vdim)))
        return out

    def new_state(self, num_slots: int) -> RecurrentStatePool:
        return RecurrentStatePool(self.state_fields(), num_slots, self.device)

    def bytes_per_state_slot(self) -> int:
        return RecurrentStatePool.bytes_per_slot(self.state_fields())

    # ------------------------------------------------------------------ forward
    def _bmm32(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """Batched a @ b with an fp32 result."""
        if self.dtype == torch.float32:
            return torch.bmm(a, b)
        if self._mm32:
            return torch.bmm(a, b, out_dtype=torch.float32)
        return torch.bmm(a.float(), b.float())

    def _latent_mixer(self, h, L: LimatarLayer, m, ri: int, positions, slots, cache, plan: StepAttention) -> torch.Tensor:
        x, T, dt = L.extra, h.shape[0], self.dtype
        C, R, D, H = m.kv_rank, m.rot_dim, m.dim, m.heads
        ci = self.cache_index[ri]
        Dk, Cv = self.latent_row_sizes(m)
        proj = self._linear(h, L.w_in)
        cq = res32.latent_kv_write(proj, m.q_rank, C, R, x["dq_norm"], x["dkv_norm"], x["freq"], x["rot_mult"], positions,
                                   slots, cache.k[ci], cache.v[ci], self.cfg.norm_eps)
        q = self._linear(cq, x["w_uq"])                                            # [T, H (D + R)]
        n_dec = plan.n_dec
        wide = T > n_dec and self.expanded_head_sizes(m) is not None and cache.block_size & (cache.block_size - 1) == 0
        n_abs = n_dec if wide else T   # rows that attend over the cached latent rows themselves
        a = torch.empty(T, H * m.vdim, dtype=dt, device=self.device)
        z, kc, vc = self._no_bias(H), cache.k[ci], cache.v[ci]
        if n_abs:
            qa, pa = q[:n_abs], positions[:n_abs]
            qn = self._bmm32(qa.view(n_abs, H, D + R)[:, :, :D].transpose(0, 1), x["w_uk"])  # [H, n, C]: keys' up-projection on q
            qf = res32.latent_q_rows(qa, D, R, qn, x["freq"], x["rot_mult"], m.scale, pa, H, Dk).view(n_abs, H * Dk)
            oc = torch.empty(n_abs, H * Cv, dtype=dt, device=self.device)
            if n_dec:
                res32.window_attn(qf[:n_dec], kc, vc, pa[:n_dec], plan.dec_tables, z, z, UNBOUNDED, oc[:n_dec], H, 1,
                                  cores=True, sink=x["sink"], values_in_keys=True)
            if n_abs > n_dec:
                ch = plan.chunk
                res32.window_attn(qf[n_dec:], kc, vc, pa[n_dec:], ch["block_tables"], z, z, UNBOUNDED, oc[n_dec:], H, 1,
                                  cu_q=ch["cu_q"], k_lens=ch.get("k_lens"), max_q=int(ch.get("max_q", 0)), cores=True,
                                  sink=x["sink"])
            o = torch.bmm(oc.view(n_abs, H, Cv)[:, :, :C].transpose(0, 1), x["w_uv_t"])      # [H, n, Dv]
            a[:n_abs] = o.transpose(0, 1).reshape(n_abs, H * m.vdim)
        if wide:
            a[n_dec:] = self._expanded_attention(q[n_dec:], positions[n_dec:], L, m, kc, cache.block_size, plan)
        res32.gate_mul(a, proj[:, m.q_rank + C + R:], "sigmoid")
        return a

    def _context_rows(self, plan: StepAttention, bs: int) -> dict:
        """For the prompt portions of a step: where every token of their sequences (the keys they may see) lies in the
        paged cache, and a dense page numbering of those tokens, sequence after sequence (built once per step)."""
        ctx = plan.scratch.get("ctx")
        if ctx is None:
            ch = plan.chunk
            k_lens = np.asarray(ch["lens"][1], dtype=np.int64)
            pages = -(-k_lens // bs)
            first = np.concatenate([[0], np.cumsum(pages)])
            item = np.repeat(np.arange(len(k_lens)), k_lens)
            pos = np.concatenate([np.arange(n) for n in k_lens]) if len(k_lens) else np.zeros(0, np.int64)
            dev = self.device
            item_d, pos_d = torch.from_numpy(item).to(dev), torch.from_numpy(pos).to(dev)
            blk = ch["block_tables"][item_d, pos_d // bs].long()
            tables = np.zeros((len(k_lens), max(1, int(pages.max()))), np.int32)
            for i, n in enumerate(pages):
                tables[i, :n] = first[i] + np.arange(n)
            ctx = plan.scratch["ctx"] = {"blk": blk, "off": pos_d % bs, "slots": torch.from_numpy(first[item] * bs + pos).to(dev),
                                         "tables": torch.from_numpy(tables).to(dev), "pages": int(first[-1])}
        return ctx

    def _expanded_attention(self, q, positions, L: LimatarLayer, m, k_rows, bs: int, plan: StepAttention) -> torch.Tensor:
        """Prompt portions over keys and values up-projected from the cached latents of their sequences: per head the
        key [W_uk c | rotated part] and the value W_uv c, laid out as pages of their own for the portion kernel."""
        x, Tq = L.extra, q.shape[0]
        C, R, D, H, Dv = m.kv_rank, m.rot_dim, m.dim, m.heads, m.vdim
        dk, dv = self.expanded_head_sizes(m)
        ctx = self._context_rows(plan, bs)
        rows = k_rows[ctx["blk"], ctx["off"]]                                      # [N, row]: latent | rotated part
        N = rows.shape[0]
        kv = F.linear(rows[:, :C], x["w_ukv"])                                     # [N, H D + H Dv]
        key = ("pages", H * dk, H * dv)
        tmp = plan.scratch.get(key)
        if tmp is None:
            tmp = plan.scratch[key] = PagedLayerCache([(H * dk, H * dv)], ctx["pages"], bs, self.device, self.dtype)
        res32.latent_expand_write(kv, rows, C, R, ctx["slots"], tmp.k[0], tmp.v[0], H, D, Dv)
        qf = res32.latent_q_rows(q, D, R, None, x["freq"], x["rot_mult"], m.scale, positions, H, dk)
        out = torch.empty(Tq, H * dv, dtype=self.dtype, device=self.device)
        ch, z = plan.chunk, self._no_bias(H)
        res32.window_attn(qf.view(Tq, H * dk), tmp.k[0], tmp.v[0], positions, ctx["tables"], z, z, UNBOUNDED, out, H, H,
                          cu_q=ch["cu_q"], k_lens=ch["k_lens"], max_q=int(ch["max_q"]), cores=True, sink=x["sink"])
        return out if dv == Dv else out.view(Tq, H, dv)[:, :, :Dv].reshape(Tq, H * Dv)

    def _retention_mixer(self, h, L: LimatarLayer, m, ri: int, state, items) -> torch.Tensor:
        x, T = L.extra, h.shape[0]
        proj = self._linear(h, L.w_in)
        nq, nv = m.nq, m.nv
        o = res32.retention(proj, nq, proj[:, 2 * nq:2 * nq + nv], x["freq"], x["rot_mult"], m.rot.dims, x["decay"],
                            state[f"S.{ri}"], items, m.heads)
        a = torch.empty(T, nv, dtype=self.dtype, device=self.device)
        res32.head_norm_gate(o, a, m.heads, self.cfg.norm_eps, w=None, gate=proj[:, 2 * nq + nv:], mode="silu")
        return a

    def _feed_forward(self, h2: torch.Tensor, L: LimatarLayer, e) -> torch.Tensor:
        x = L.extra
        if isinstance(e, ClampedGluSpec):
            act = res32.glu(self._linear(h2, x["w_gu"]), mode="clamped", alpha=e.alpha, limit=e.limit)
            return self._linear(act, x["w_down"])
        if "router_t" in x:   # bf16 operands, fp32 accumulation AND output: the checkpoint's router is bf16-exact
            z = torch.mm(h2, x["router_t"], out_dtype=torch.float32)
        else:
            z = F.linear(h2.float(), x["router"])
        _ids, w, row_off, src, row_expert, inv = res32.router(z, None, e.experts, e.top, bias=x["router_b"], renorm=True)
        d = self.cfg.hidden
        if (self.dtype == torch.bfloat16 and d * e.ff >= self.GROUPED_MIN and d % 64 == 0 and e.ff % 64 == 0
                and ops.available()):
            gu = ops.grouped_gemm(h2, x["w_gu"], row_off, a_rows=src, rows=src.numel())
            Y = ops.grouped_gemm(res32.glu(gu), x["w_down"], row_off)
        else:
            Y = res32.expert_rows(h2, src, row_expert, row_off, x["w_gu"], x["w_down"])
        shared = None
        if e.shared_ff:
            shared = self._linear(res32.glu(self._linear(h2, x["ws_gu"])), x["ws_down"])
        return res32.moe_combine(Y, inv, w, h2, add=shared)

    def _forward(self, tokens, positions, slots, cache: PagedLayerCache, state: RecurrentStatePool,
                 items: res32.StepItems, plan: StepAttention, keep: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Every layer run over the step's rows; ``plan`` says how the rows reach the paged cache.
        Returns the fp32 stream that the output norm reads, [T, d].

        ``keep`` (int64 rows): only these rows' final states are wanted (a prompt's last token).  The LAST run then
        still runs its mixer on every row (the cached rows and the recurrent state are what later steps read) but the
        output projection and the feed-forward on the kept rows only; returns [len(keep), d]."""
        cfg, dt, eps = self.cfg, self.dtype, self.cfg.norm_eps
        x = res32.rmsnorm_rows(res32.embed_rows(self.embed, tokens), self.embed_norm, eps, torch.float32)
        n = len(self.runs)
        h = res32.rmsnorm_rows(x, self.layers[self.runs[0]].norm1, eps, dt) if n else None
        for ri, li in enumerate(self.runs):
            S, L = cfg.layer_specs[li], self.layers[li]
            if S.type == "latent_attention":
                a = self._latent_mixer(h, L, S.mixer, ri, positions, slots, cache, plan)
            else:
                a = self._retention_mixer(h, L, S.mixer, ri, state, items)
            last = ri + 1 == n
            if keep is not None and last:   # from here on only the kept rows
                a, x = a.index_select(0, keep), x.index_select(0, keep)
            nxt = None if last else self.layers[self.runs[ri + 1]].norm1
            y = self._linear(a, L.w_o)
            if S.mlp is not None:
                h2 = self._add_norm(x, y, L.norm1b, L.norm2)
                h = self._add_norm(x, self._feed_forward(h2, L, S.mlp), L.norm2b, nxt)
            else:
                h = self._add_norm(x, y, L.norm1b, nxt)
            if self.on_layer is not None:
                self.on_layer(ri, x)
        return x

    def _add_norm(self, x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, next_w: Optional[torch.Tensor]):
        """x += y / rms(y) * w; returns the next sublayer's input x / rms(x) * next_w (None without ``next_w``): one
        pass over the stream in bf16 (the new x stays in registers between the two norms)."""
        eps = self.cfg.norm_eps
        if next_w is None:
            res32.gated_norm_residual(x, y, w, eps)
            return None
        if self.dtype == torch.bfloat16:
            h = torch.empty(x.shape[0], x.shape[1], dtype=self.dtype, device=self.device)
            res32.gated_norm_residual(x, y, w, eps, x_cast=h, next_w=next_w)
            return h
        res32.gated_norm_residual(x, y, w, eps)
        return res32.rmsnorm_rows(x, next_w, eps, self.dtype)

    def _logits(self, x: torch.Tensor, rows: Optional[torch.Tensor], float_logits: bool) -> torch.Tensor:
        h = res32.rmsnorm_rows(x, self.final_w, self.cfg.norm_eps, self.dtype, rows=rows)
        lg = self._linear(h, self.embed).float()
        if float_logits:
            return lg
        V, Vp = self.cfg.vocab_size, self.logit_width
        if Vp == V:
            return lg.to(torch.bfloat16)
        out = torch.full((lg.shape[0], Vp), float("-inf"), dtype=torch.bfloat16, device=lg.device)
        out[:, :V] = lg
        return out

    def _no_bias(self, H: int) -> torch.Tensor:
        z = self._zeros_h.get(H)
        if z is None:
            z = self._zeros_h[H] = torch.zeros(H, dtype=torch.float32, device=self.device)
        return z

    def decode(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, block_tables: torch.Tensor,
               ctx_lens: torch.Tensor, cache: PagedLayerCache, num_splits: int = 1, cascade_tiles=None,
               float_logits: bool = False, state: Optional[RecurrentStatePool] = None,
               state_slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One decode step for B sequences -> logits [B, V]; device tensors only (hipGraph-capturable).  Row b
        reads table row b and the state slot ``state_slots[b]``; its key range ends at its own position."""
        if state is None or state_slots is None:
            raise RuntimeError("Limatar: a decode step needs the recurrent-state pool and the rows' slots")
        items = res32.StepItems.rows(state_slots, positions)
        x = self._forward(tokens, positions, slots, cache, state, items, StepAttention(tokens.shape[0], block_tables, None))
        return self._logits(x, None, float_logits)

    def forward_mixed(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, cache: PagedLayerCache,
                      n_dec: int, dec: Optional[dict], chunk: Optional[dict], logit_rows: torch.Tensor,
                      float_logits: bool = False, state: Optional[RecurrentStatePool] = None,
                      state_slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """ONE forward over [n_dec decode rows || prompt-portion rows]: every projection is one GEMM over both, the
        recurrence walks decode rows and portions alike as items; the attention runs per part over the paged cache
        that this step's rows were just written to.  ``state_slots``: int32, the slot of every decode row, then of
        every portion.  Logits of ``logit_rows``."""
        if state is None or state_slots is None:
            raise RuntimeError("Limatar: a step needs the recurrent-state pool and the sequences' slots")
        T = tokens.shape[0]
        q_lens = list(chunk["lens"][0]) if T > n_dec else []
        cu = np.concatenate([np.arange(n_dec, dtype=np.int64), n_dec + np.concatenate([[0], np.cumsum(q_lens, dtype=np.int64)])])
        if cu[-1] != T or state_slots.numel() != n_dec + len(q_lens):
            raise ValueError("Limatar: rows, portions and state slots disagree")
        row_item = np.concatenate([np.arange(n_dec, dtype=np.int64), n_dec + np.repeat(np.arange(len(q_lens)), q_lens)])
        dev = self.device
        items = res32.StepItems(torch.from_numpy(row_item.astype(np.int32)).to(dev), torch.from_numpy(cu.astype(np.int32)).to(dev),
                                state_slots, positions)
        plan = StepAttention(n_dec, dec["block_tables"] if n_dec else None, chunk if T > n_dec else None)
        keep = logit_rows if n_dec == 0 and self.on_layer is None and 4 * logit_rows.numel() <= T else None
        x = self._forward(tokens, positions, slots, cache, state, items, plan, keep=keep)
        return self._logits(x, None if keep is not None else logit_rows, float_logits)

    def prefill(self, tokens, positions, slots, cu_seqlens, max_seqlen, last_idx, cache, ctx=None):
        raise RuntimeError("Limatar prefills through forward_mixed over the paged cache (paged_prefill)")
