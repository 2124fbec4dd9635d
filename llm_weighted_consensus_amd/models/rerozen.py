"""Rerozen decoder on the fp32-residual kernel set (``ops/res32.py``, ``csrc/kernels/res32``).

The residual stream x is fp32, layers are pre-norm.  A layer over the T rows of a step (decode rows and prompt-portion
rows alike); every mixer is TWO mixers on the same input whose results are added with fixed scales:

    n      = x / rms(x) * w1  (fp32)                   res32.add_rmsnorm (with the residual add of the sublayer before)
    h      = n + conv_t(n)                              res32.conv_hist (per-sequence history slot)
    proj   = h @ [left q|k|v|g  right q|k|v|...|a1]^T   ONE GEMM (+ the left biases)
    left, a chunked rotary attention:
      qkv  = conv_t(proj_qkv)                           res32.conv_hist, no activation ("parallel_2" only; history slot)
      q    = rot(norm(q)) * scale;  cache <- rot(norm(k)), v or rot(v)      res32.rot_kv_write
      o    = softmax over the keys of the row's own chunk (a sink of score 0 in "parallel_2")   res32.window_attn
      a_l  = unrot(o) * sigmoid(g_h) * left_scale       res32.head_gate_unrotate
    right, a linear attention with a decay per head and key channel (state fp32 [H, D, Dv] in the state slot):
      z    = a1 @ Wa2^T                                 GEMM, fp32 result
      "parallel":   S <- diag(sigmoid(z + b)^(1/tau)) S + k v^T;  o = S^T q                    res32.channel_decay_rule
                    a_r = o / rms(o) * w * silu(proj_g) * right_scale                          res32.head_norm_gate
      "parallel_2": q, k, v = silu(conv_t(.)) (history slot), unit q / k, gated delta rule with the decays
                    exp(-exp(A_log) softplus(z + dt_bias));  a_r = o / rms(o) * w * sigmoid(g1 @ Wg2^T) * right_scale
    y      = [a_l | a_r] @ [Wo_left | Wo_right]^T       ONE GEMM: both mixers' output projections summed in the GEMM
    n2     = norm2(x += y);  h2 = n2 + conv_t(n2)       res32.add_rmsnorm, res32.conv_hist
    x     += gelu(h2 @ Wup^T) @ Wdown^T                 res32.gelu (erf form)

Logits = (norm(x) @ head^T) * logit_scale; the embedding is scaled by ``embed_scale``.  Per-sequence state besides the
K/V pages lives in a :class:`..models.state.RecurrentStatePool` whose slots the engine's block manager hands out.
``dtype=torch.float32`` runs every GEMM, activation and the cache in true fp32; bf16 is the serving mode.
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
from .config import RerozenConfig
from .state import RecurrentStatePool

UNBOUNDED = 1 << 30  # "window" of an attention whose only bound is its chunk


@dataclass
class RerozenLayer:
    norm1: torch.Tensor                  # fp32
    canon1: torch.Tensor                 # fp32 [d, taps], tap-major storage
    w_in: torch.Tensor                   # every input-side projection of both mixers, fused
    b_in: Optional[torch.Tensor]
    w_o: torch.Tensor                    # [d, H Dv (left) + H Dv (right)]
    cols: Dict[str, slice]               # columns of the fused projection
    norm2: Optional[torch.Tensor] = None
    canon2: Optional[torch.Tensor] = None
    w_up: Optional[torch.Tensor] = None
    w_down: Optional[torch.Tensor] = None
    extra: Dict[str, object] = field(default_factory=dict)


class RerozenModel:
    paged_prefill = True      # whole prompts run as one portion over the paged cache (engine._run_prefill)
    supports_cascade = False
    graph_safe = True
    float_logits = True
    has_state = True          # the engine gives every sequence a recurrent-state slot

    def __init__(self, cfg: RerozenConfig, device="cuda", dtype=torch.bfloat16, seed: int = 0,
                 weights_path: Optional[str] = None, max_position: Optional[int] = None):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Rerozen runs in bfloat16 or float32")
        self.device, self.dtype = torch.device(device), dtype
        if self.device.type != "cuda":
            raise RuntimeError("Rerozen runs on the GPU kernels only (no CPU path)")
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False
        raw = None
        if weights_path:
            raw = self._read_files(weights_path)
            cfg = cfg.with_ranks({k: tuple(v.shape) for k, v in raw.items()})
        self.cfg = cfg
        K = res32.kernels()
        if not 1 <= cfg.canon_taps <= 16:
            raise ValueError("Rerozen: canon.taps must be in 1..16")
        for L in cfg.layer_specs:
            if L.right.dim > K.chan_rule_max_dim() or L.left.conv > 16 or L.right.conv > 16 or L.left.vdim > 512:
                raise ValueError("Rerozen: mixer sizes beyond what the kernels are built for")
            if L.right.a_rank < 1 or (L.right.kind == "delta" and L.right.g_rank < 1):
                raise ValueError("Rerozen: the low-rank widths come from a checkpoint or the config (a_rank, g_rank)")
        self.logit_width = -(-cfg.vocab_size // 32) * 32
        self._mm32 = self._probe_mm32()
        if raw is None:
            raw = self._random(seed)
        else:
            self._check(raw, weights_path)
        self._assemble(raw)
        self.g8_ws = None
        self.on_layer: Optional[Callable[[int, torch.Tensor], None]] = None
        self._zeros_h: Dict[int, torch.Tensor] = {}

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self) -> dict:
        """name -> shape of every tensor of a checkpoint of this config."""
        cfg, d = self.cfg, self.cfg.hidden
        out = {"embed": (cfg.vocab_size, d), "final.norm": (d,), "head": (cfg.vocab_size, d)}
        for i, L in enumerate(cfg.layer_specs):
            a, r = L.left, L.right
            p, pl, pr = f"l{i}.", f"l{i}.mix.left.", f"l{i}.mix.right."
            out.update({p + "norm1": (d,), p + "canon1": (d, cfg.canon_taps)})
            out.update({pl + "q": (a.nq, d), pl + "k": (a.nk, d), pl + "v": (a.nv, d), pl + "g": (a.heads, d),
                        pl + "o": (d, a.heads * a.vdim)})
            if a.bias:
                out.update({pl + "q.b": (a.nq,), pl + "k.b": (a.nk,), pl + "v.b": (a.nv,)})
            if a.qk_norm:
                out.update({pl + "q.norm": (a.dim,), pl + "k.norm": (a.dim,)})
            if a.conv:
                out.update({pl + "q.conv": (a.nq, a.conv), pl + "k.conv": (a.nk, a.conv), pl + "v.conv": (a.nv, a.conv)})
            out.update({pr + "q": (r.nq, d), pr + "k": (r.nq, d), pr + "v": (r.nv, d), pr + "o": (d, r.nv), pr + "norm": (r.vdim,),
                        pr + "a1": (r.a_rank, d), pr + "a2": (r.nd, r.a_rank)})
            if r.kind == "delta":
                out.update({pr + "q.conv": (r.nq, r.conv), pr + "k.conv": (r.nq, r.conv), pr + "v.conv": (r.nv, r.conv),
                            pr + "b": (r.heads, d), pr + "A_log": (r.heads,), pr + "dt_bias": (r.nd,),
                            pr + "g1": (r.g_rank, d), pr + "g2": (r.nv, r.g_rank)})
            else:
                out.update({pr + "g": (r.nv, d), pr + "a2.b": (r.nd,)})
            if L.ff:
                out.update({p + "norm2": (d,), p + "canon2": (d, cfg.canon_taps), p + "mlp.up": (L.ff, d),
                            p + "mlp.down": (d, L.ff)})
        return out

    def _random(self, seed: int) -> dict:
        """Random weights of the config's shapes (benchmarks, tests): bf16-representable values."""
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        d = self.cfg.hidden
        out = {}
        for name, shape in self.tensor_shapes().items():
            leaf = name.split(".")[-1]
            if leaf in ("norm1", "norm2", "norm"):
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            elif leaf in ("canon1", "canon2"):
                t = 0.2 * torch.randn(shape, generator=g)
            elif leaf == "conv":
                t = 0.5 * torch.randn(shape, generator=g)
            elif leaf == "b" and len(shape) == 1:
                t = 0.1 * torch.randn(shape, generator=g)
            elif leaf == "A_log":
                t = torch.rand(shape, generator=g) * 2 - 1
            elif leaf == "dt_bias":
                t = torch.randn(shape, generator=g)
            elif name == "embed":
                t = torch.randn(shape, generator=g) / math.sqrt(d)
            else:
                t = torch.randn(shape, generator=g) / math.sqrt(shape[-1] if len(shape) > 1 else d)
            out[name] = t.to(torch.bfloat16)
        return out

    @staticmethod
    def _read_files(path: str) -> dict:
        from safetensors.torch import load_file

        p = Path(path)
        files = sorted(p.glob("*.safetensors")) if p.is_dir() else [p]
        if not files:
            raise FileNotFoundError(f"no .safetensors under {path}")
        sd = {}
        for f in files:
            sd.update(load_file(str(f), device="cpu"))
        return sd

    def _check(self, sd: dict, path: str) -> None:
        for name, shape in self.tensor_shapes().items():
            if name not in sd:
                raise KeyError(f"{path}: tensor {name} missing")
            if tuple(sd[name].shape) != tuple(shape):
                raise ValueError(f"{path}: {name} has shape {tuple(sd[name].shape)}, the config says {tuple(shape)}")

    def _assemble(self, sd: dict) -> None:
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def t(name):
            return sd[name].to(device=dev, dtype=dt).contiguous()

        def f32(name):
            return sd[name].to(device=dev, dtype=torch.float32).contiguous()

        def taps_major(w):
            """[C, taps] convolution weights stored tap-major (the kernels' 16-byte path reads w[j][c : c + 4])."""
            return w.t().contiguous().t()

        self.embed, self.head, self.final_w = t("embed"), t("head"), f32("final.norm")
        self.layers: List[RerozenLayer] = []
        for i, L in enumerate(cfg.layer_specs):
            a, r = L.left, L.right
            p, pl, pr = f"l{i}.", f"l{i}.mix.left.", f"l{i}.mix.right."
            parts = [("lq", pl + "q"), ("lk", pl + "k"), ("lv", pl + "v"), ("lg", pl + "g"), ("rq", pr + "q"), ("rk", pr + "k"),
                     ("rv", pr + "v")]
            parts += [("rb", pr + "b"), ("a1", pr + "a1"), ("g1", pr + "g1")] if r.kind == "delta" else [("rg", pr + "g"), ("a1", pr + "a1")]
            cols, o, ws = {}, 0, []
            for key, name in parts:
                w = t(name)
                cols[key] = slice(o, o + w.shape[0])
                o += w.shape[0]
                ws.append(w)
            cols["lqkv"] = slice(cols["lq"].start, cols["lv"].stop)
            cols["rqkv"] = slice(cols["rq"].start, cols["rv"].stop)
            w_in = torch.cat(ws, 0).contiguous()
            b_in = None
            if a.bias:
                b_in = torch.zeros(o, dtype=dt, device=dev)
                b_in[cols["lqkv"]] = torch.cat([t(pl + "q.b"), t(pl + "k.b"), t(pl + "v.b")])
            x: Dict[str, object] = {}
            x["freq"], x["rot_mult"] = res32.rope_frequencies(a.rot.dims, a.rot.base, a.rot.scaling_dict(), dev) if a.rot.dims else (None, 1.0)
            x["vfreq"] = res32.rope_frequencies(a.vdim, a.rot.base, None, dev)[0] if a.rotate_values else None
            x["wq"], x["wk"] = (f32(pl + "q.norm"), f32(pl + "k.norm")) if a.qk_norm else (None, None)
            if a.conv:
                x["lconv"] = taps_major(torch.cat([f32(pl + "q.conv"), f32(pl + "k.conv"), f32(pl + "v.conv")], 0))
            x["sink"] = torch.zeros(a.heads, dtype=torch.float32, device=dev) if a.sink else None   # exp(0) = the added one
            # the right mixer's per-head norm weight carries the mixer's fixed scale
            x["rnorm"] = (f32(pr + "norm") * L.right_scale).contiguous()
            x["w_a2"] = self._small(sd[pr + "a2"])
            if r.kind == "delta":
                x["rconv"] = taps_major(torch.cat([f32(pr + "q.conv"), f32(pr + "k.conv"), f32(pr + "v.conv")], 0))
                x["A_log"], x["zb"] = f32(pr + "A_log"), f32(pr + "dt_bias")
                x["w_g2"] = t(pr + "g2")
            else:
                x["zb"] = f32(pr + "a2.b")
            lay = RerozenLayer(norm1=f32(p + "norm1"), canon1=taps_major(f32(p + "canon1")), w_in=w_in, b_in=b_in,
                               w_o=torch.cat([t(pl + "o"), t(pr + "o")], 1).contiguous(), cols=cols, extra=x)
            if L.ff:
                lay.norm2, lay.canon2 = f32(p + "norm2"), taps_major(f32(p + "canon2"))
                lay.w_up, lay.w_down = t(p + "mlp.up"), t(p + "mlp.down")
            self.layers.append(lay)

    def _small(self, w: torch.Tensor):
        """The second matrix of a low-rank pair whose product enters a recurrence: kept so that the product comes out in
        fp32 (bf16 operands with an fp32 result where this torch build has that, else fp32 operands)."""
        if self._mm32:
            return w.to(device=self.device, dtype=self.dtype).t().contiguous()      # [rank, out]
        return w.to(device=self.device, dtype=torch.float32).contiguous()           # [out, rank]

    # ------------------------------------------------------------------ GEMMs
    def _probe_mm32(self) -> bool:
        """Whether this torch build multiplies bf16 matrices into an fp32 result (the decay logits)."""
        if self.dtype != torch.bfloat16:
            return False
        try:
            a = torch.zeros(8, 16, dtype=self.dtype, device=self.device)
            return torch.mm(a, a.t(), out_dtype=torch.float32).dtype == torch.float32
        except (TypeError, RuntimeError):
            return False

    def _linear(self, x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
        if b is None and self.g8_ws is not None:
            return gemm_plan.linear(x, w, ws=self.g8_ws)
        return F.linear(x, w, b)

    def _decay_logits(self, a1: torch.Tensor, w) -> torch.Tensor:
        """a1 @ W^T with an fp32 result ([T, H D])."""
        if self._mm32:
            return torch.mm(a1, w, out_dtype=torch.float32)
        return F.linear(a1.float(), w)

    def tune_gemms(self, M: int, bucket: bool = False, lm_head: bool = True, only=None) -> None:
        """Pick the backend of the bias-free projections at M rows by timing the library and the hand-written cores (the
        engine calls this before it captures a decode bucket's graph).  bf16 only, and only where the full kernel
        extension is built; otherwise every GEMM stays on the library."""
        if self.dtype != torch.bfloat16 or only is not None or not ops.available():
            return
        if self.g8_ws is None:
            self.g8_ws = ops.new_gemm8p_workspace(self.device)
        seen = set()
        ws = [w for L in self.layers for w in (L.w_o, L.w_up, L.w_down, L.w_in if L.b_in is None else None)]
        for w in ws + ([self.head] if lm_head else []):
            if w is not None and tuple(w.shape) not in seen and w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0:
                seen.add(tuple(w.shape))
                gemm_plan.tune(torch.randn(M, w.shape[1], device=self.device).to(self.dtype), w, ws=self.g8_ws, bucket=bucket)

    # ------------------------------------------------------------------ cache and state
    def _layer_dims(self):
        return [(L.left.nk, L.left.nv) for L in self.cfg.layer_specs]

    def new_cache(self, num_blocks: int, block_size: int) -> PagedLayerCache:
        return PagedLayerCache(self._layer_dims(), num_blocks, block_size, self.device, self.dtype)

    def bytes_per_block(self, block_size: int) -> int:
        n = PagedLayerCache.elems_per_block(self._layer_dims(), block_size) * (4 if self.dtype == torch.float32 else 2)
        return max(n, 16)

    def state_fields(self):
        """(name, shape) of every per-sequence state tensor: per layer the input convolutions' last inputs of both
        sublayers, the short convolutions' last inputs of either mixer, and the linear attention's matrices."""
        cfg, d, k = self.cfg, self.cfg.hidden, self.cfg.canon_taps - 1
        out = []
        for i, L in enumerate(cfg.layer_specs):
            a, r = L.left, L.right
            out.append((f"c1.{i}", (k, d)))
            if L.ff:
                out.append((f"c2.{i}", (k, d)))
            if a.conv:
                out.append((f"lc.{i}", (a.conv - 1, a.nq + a.nk + a.nv)))
            if r.kind == "delta":
                out.append((f"rc.{i}", (r.conv - 1, 2 * r.nq + r.nv)))
            out.append((f"S.{i}", (r.heads, r.dim, r.vdim)))
        return out

    def new_state(self, num_slots: int) -> RecurrentStatePool:
        return RecurrentStatePool(self.state_fields(), num_slots, self.device)

    def bytes_per_state_slot(self) -> int:
        return RecurrentStatePool.bytes_per_slot(self.state_fields())

    # ------------------------------------------------------------------ forward
    def _left(self, proj, L: RerozenLayer, a, li: int, positions, slots, cache, state, items, attend, out, scale: float):
        """The chunked rotary attention of layer ``li`` -> ``out`` (a column slice of the output GEMM's input)."""
        x, T = L.extra, proj.shape[0]
        qkv = proj[:, L.cols["lqkv"]]
        if a.conv:
            raw, qkv = qkv, torch.empty(T, a.nq + a.nk + a.nv, dtype=torch.float32, device=self.device)
            res32.conv_hist(raw, x["lconv"], state[f"lc.{li}"], items, qkv, mode=2)
        q = res32.rot_kv_write(qkv, positions, slots, cache.k[li], cache.v[li], a.heads, a.kv_heads, a.scale,
                               rot_dims=a.rot.dims, freq=x["freq"], mult=x["rot_mult"], vfreq=x["vfreq"], wq=x["wq"], wk=x["wk"],
                               eps=self.cfg.norm_eps)
        o = torch.empty(T, a.heads * a.vdim, dtype=self.dtype, device=self.device)
        attend(q, li, o)
        res32.head_gate_unrotate(o, out, positions, a.heads, gate=proj[:, L.cols["lg"]], vfreq=x["vfreq"], scale=scale)

    def _right(self, proj, L: RerozenLayer, r, li: int, state, items, out):
        """The channel-decay linear attention of layer ``li`` -> ``out``."""
        x, T, eps = L.extra, proj.shape[0], self.cfg.norm_eps
        z = self._decay_logits(proj[:, L.cols["a1"]], x["w_a2"])
        S = state[f"S.{li}"]
        if r.kind == "delta":
            qkv = torch.empty(T, 2 * r.nq + r.nv, dtype=torch.float32, device=self.device)
            res32.conv_hist(proj[:, L.cols["rqkv"]], x["rconv"], state[f"rc.{li}"], items, qkv, mode=1)
            o = res32.channel_decay_rule(qkv, z, S, items, r.heads, r.kv_heads, zb=x["zb"], A_log=x["A_log"],
                                         beta=proj[:, L.cols["rb"]], unit=True, delta=True)
            gate = self._linear(proj[:, L.cols["g1"]], x["w_g2"])
            res32.head_norm_gate(o, out, r.heads, eps, w=x["rnorm"], gate=gate, mode="sigmoid")
        else:
            o = res32.channel_decay_rule(proj[:, L.cols["rqkv"]], z, S, items, r.heads, r.kv_heads, zb=x["zb"], tau=r.tau)
            res32.head_norm_gate(o, out, r.heads, eps, w=x["rnorm"], gate=proj[:, L.cols["rg"]], mode="silu")

    def _forward(self, tokens, positions, slots, cache: PagedLayerCache, state: RecurrentStatePool,
                 items: res32.StepItems, attend) -> torch.Tensor:
        """Every layer over the step's rows; ``attend(q, li, out)`` runs the attention of layer ``li`` into ``out``.
        Returns the fp32 stream that the output norm reads, [T, d]."""
        cfg, dt, dev = self.cfg, self.dtype, self.device
        T, d, eps, nl = tokens.shape[0], cfg.hidden, cfg.norm_eps, len(self.layers)
        x = res32.embed_rows(self.embed, tokens, scale=cfg.embed_scale)
        n = res32.add_rmsnorm(x, None, self.layers[0].norm1, eps, torch.float32) if nl else None
        h = torch.empty(T, d, dtype=dt, device=dev)
        for li, (S, L) in enumerate(zip(cfg.layer_specs, self.layers)):
            a, r = S.left, S.right
            res32.conv_hist(n, L.canon1, state[f"c1.{li}"], items, h, mode=0)
            proj = self._linear(h, L.w_in, L.b_in)
            nl_cols = a.heads * a.vdim
            cat = torch.empty(T, nl_cols + r.nv, dtype=dt, device=dev)
            self._left(proj, L, a, li, positions, slots, cache, state, items, attend, cat[:, :nl_cols], S.left_scale)
            self._right(proj, L, r, li, state, items, cat[:, nl_cols:])
            y = self._linear(cat, L.w_o)
            if S.ff:
                res32.add_rmsnorm(x, y, L.norm2, eps, torch.float32, out=n)
                res32.conv_hist(n, L.canon2, state[f"c2.{li}"], items, h, mode=0)
                y = self._linear(res32.gelu(self._linear(h, L.w_up)), L.w_down)
            if li + 1 < nl:
                res32.add_rmsnorm(x, y, self.layers[li + 1].norm1, eps, torch.float32, out=n)
            else:
                res32.residual_add_scaled(x, y, 1.0)
            if self.on_layer is not None:
                self.on_layer(li, x)
        return x

    def _logits(self, x: torch.Tensor, rows: Optional[torch.Tensor], float_logits: bool) -> torch.Tensor:
        h = res32.rmsnorm_rows(x, self.final_w, self.cfg.norm_eps, self.dtype, rows=rows)
        lg = self._linear(h, self.head).float() * self.cfg.logit_scale
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

    def _attend(self, cache, positions, tables, cu_q=None, k_lens=None, max_q=0):
        def run(q, li, out, rows=slice(None)):
            a = self.cfg.layer_specs[li].left
            z = self._no_bias(a.heads)
            res32.window_attn(q[rows], cache.k[li], cache.v[li], positions[rows], tables, z, z, UNBOUNDED, out[rows],
                              a.heads, a.kv_heads, cu_q=cu_q, k_lens=k_lens, max_q=max_q, bias=None, cores=True,
                              sink=self.layers[li].extra["sink"], chunk=a.chunk)
        return run

    def decode(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, block_tables: torch.Tensor,
               ctx_lens: torch.Tensor, cache: PagedLayerCache, num_splits: int = 1, cascade_tiles=None,
               float_logits: bool = False, state: Optional[RecurrentStatePool] = None,
               state_slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One decode step for B sequences -> logits [B, V]; device tensors only (hipGraph-capturable).  Row b
        reads table row b and the state slot ``state_slots[b]``; its key range ends at its own position."""
        if state is None or state_slots is None:
            raise RuntimeError("Rerozen: a decode step needs the recurrent-state pool and the rows' slots")
        items = res32.StepItems.rows(state_slots, positions)
        x = self._forward(tokens, positions, slots, cache, state, items, self._attend(cache, positions, block_tables))
        return self._logits(x, None, float_logits)

    def forward_mixed(self, tokens: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, cache: PagedLayerCache,
                      n_dec: int, dec: Optional[dict], chunk: Optional[dict], logit_rows: torch.Tensor,
                      float_logits: bool = False, state: Optional[RecurrentStatePool] = None,
                      state_slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """ONE forward over [n_dec decode rows || prompt-portion rows]: every projection is one GEMM over both, the
        convolutions and the recurrences walk decode rows and portions alike as items; the attention runs per part over
        the paged cache that this step's rows were just written to.  ``state_slots``: int32, the slot of every decode
        row, then of every portion.  Logits of ``logit_rows``."""
        if state is None or state_slots is None:
            raise RuntimeError("Rerozen: a step needs the recurrent-state pool and the sequences' slots")
        T = tokens.shape[0]
        q_lens = list(chunk["lens"][0]) if T > n_dec else []
        cu = np.concatenate([np.arange(n_dec, dtype=np.int64), n_dec + np.concatenate([[0], np.cumsum(q_lens, dtype=np.int64)])])
        if cu[-1] != T or state_slots.numel() != n_dec + len(q_lens):
            raise ValueError("Rerozen: rows, portions and state slots disagree")
        row_item = np.concatenate([np.arange(n_dec, dtype=np.int64), n_dec + np.repeat(np.arange(len(q_lens)), q_lens)])
        dev = self.device
        items = res32.StepItems(torch.from_numpy(row_item.astype(np.int32)).to(dev), torch.from_numpy(cu.astype(np.int32)).to(dev),
                                state_slots, positions)
        dec_run = self._attend(cache, positions, dec["block_tables"]) if n_dec else None
        chk_run = (self._attend(cache, positions, chunk["block_tables"], cu_q=chunk["cu_q"], k_lens=chunk.get("k_lens"),
                                max_q=int(chunk.get("max_q", 0))) if T > n_dec else None)

        def attend(q, li, out):
            if dec_run is not None:
                dec_run(q, li, out, slice(0, n_dec))
            if chk_run is not None:
                chk_run(q, li, out, slice(n_dec, T))

        x = self._forward(tokens, positions, slots, cache, state, items, attend)
        return self._logits(x, logit_rows, float_logits)

    def prefill(self, tokens, positions, slots, cu_seqlens, max_seqlen, last_idx, cache, ctx=None):
        raise RuntimeError("Rerozen prefills through forward_mixed over the paged cache (paged_prefill)")
