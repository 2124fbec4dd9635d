#!/usr/bin/env python3
"""Prefill and decode throughput of two decoder designs at equal size, through the engine.

    python bench.py --compare-decoders [--sizes small,8b-layer] [--compare-layers 4]

Designs: ``madipel``, ``llama``, ``merudra``, ``mixtral``, ``limatar``, ``rerozen`` (``--designs merudra,mixtral`` puts Merudra
beside the closest existing decoder, the routed-experts Mixtral: 8 experts, 2 per token, the same active feed-forward
width; Merudra's layers alternate attention and gated delta rule mixers and add 2 identity experts.
``--designs limatar,merudra`` puts Limatar beside Merudra, the closest decoder with paged attention AND recurrent
layers over an fp32 stream: Limatar's layers alternate low-rank attention (latent 512 + 64 rotated entries, sinks) and
retention, routed experts with a shared expert and the clamped dense unit).
``--designs rerozen,merudra`` puts Rerozen beside Merudra, the closest decoder (input convolutions in front of every
sublayer, paged attention and gated delta rule layers over an fp32 stream): every Rerozen layer runs a chunked rotary
attention AND a half-size channel-decay linear attention side by side, and a dense gelu feed-forward).

For each size a Madipel model (parallel layers, windowed attention with distance bias, xIELU feed-forward, fp32
residual) and the closest existing decoder (Llama: sequential layers, causal GQA attention with RoPE, SwiGLU) are
built with random weights at the same width, layer count, head counts, head size, vocabulary and parameter count
(Madipel's two feed-forward matrices get 1.5x Llama's inner width to match its three), and run through the same
LLMEngine: prefill = whole prompts in one admission batch (tokens/s), decode = hipGraph decode steps of a fixed
batch at a fixed context (tokens/s).  One JSON line per (size, design) and a closing summary line.
"""
from __future__ import annotations

import json
import sys
import time

SIZES = {
    # name: width, heads, kv_heads, head_dim, llama_ffn, vocab
    "small": dict(width=2048, heads=16, kv_heads=4, head_dim=128, ffn=8192, vocab=32000),
    "8b-layer": dict(width=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, vocab=32000),
}


def _madipel(size: dict, layers: int, window: int, device, seed: int):
    from llm_weighted_consensus_amd.models.config import MadipelConfig
    from llm_weighted_consensus_amd.models.madipel import MadipelModel

    layer = {"type": "attention",
             "mixer": {"heads": size["heads"], "kv_heads": size["kv_heads"], "dim": size["head_dim"], "vdim": size["head_dim"],
                       "mask": {"size": window}, "scale": size["head_dim"] ** -0.5, "v_mix": True},
             "mlp": {"kind": "dense", "ff": size["ffn"] * 3 // 2}}
    cfg = MadipelConfig.from_dict({"architecture": "Madipel", "layers": [layer] * layers, "logit_scale": 1.0,
                                   "norm": {"eps": 1e-5}, "residual_mult": 0.5, "vocab": size["vocab"],
                                   "width": size["width"]}, name="madipel-bench")
    return MadipelModel(cfg, device=device, seed=seed)


def _llama(size: dict, layers: int, max_pos: int, device, seed: int):
    from llm_weighted_consensus_amd.models.config import DecoderConfig
    from llm_weighted_consensus_amd.models.llama import LlamaModel

    cfg = DecoderConfig("llama-bench", size["vocab"], size["width"], layers, size["heads"], size["kv_heads"],
                        size["head_dim"], size["ffn"], max_position=max_pos)
    return LlamaModel(cfg, device=device, seed=seed, max_position=max_pos)


def _merudra(size: dict, layers: int, device, seed: int, experts: int = 8, top: int = 2, pattern: str = "ad"):
    """Attention and delta layers alternating (``pattern``: a / d per layer, repeated), routed experts of inner width
    ffn / top (the active feed-forward width of the dense models), two identity experts."""
    from llm_weighted_consensus_amd.models.config import MerudraConfig
    from llm_weighted_consensus_amd.models.merudra import MerudraModel

    H, G, D = size["heads"], size["kv_heads"], size["head_dim"]
    mlp = {"kind": "moe", "expert": {"ff": size["ffn"] // top}, "router": {"experts": experts, "identity": 2, "top": top}}
    att = {"type": "attention", "mlp": mlp,
           "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "q_temp": {"coef": 0.1, "every": 512}}}
    dlt = {"type": "delta", "mlp": mlp, "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": 4}}
    cfg = MerudraConfig.from_dict({"architecture": "Merudra", "canon": {"taps": 4},
                                   "layers": [att if pattern[i % len(pattern)] == "a" else dlt for i in range(layers)],
                                   "norm": {"eps": 1e-5}, "token_side": {"dim": 64}, "vocab": size["vocab"],
                                   "width": size["width"]}, name="merudra-bench")
    return MerudraModel(cfg, device=device, seed=seed)


def _limatar(size: dict, layers: int, device, seed: int, experts: int = 8, top: int = 2, pattern: str = "lr"):
    """Low-rank attention and retention layers alternating (``pattern``: l / r per layer, repeated; a / d of the other
    designs' patterns mean the same), feed-forwards alternating in pairs between routed experts (inner width ffn / top,
    a shared expert of ffn / 8) and the dense clamped unit of inner width ffn: the same active width everywhere."""
    from llm_weighted_consensus_amd.models.config import LimatarConfig
    from llm_weighted_consensus_amd.models.limatar import LimatarModel

    H, D, d = size["heads"], size["head_dim"], size["width"]
    moe = {"kind": "moe", "expert": {"ff": size["ffn"] // top}, "router": {"experts": experts, "top": top},
           "shared": {"ff": size["ffn"] // 8}}
    dense = {"kind": "dense", "ff": size["ffn"], "limit": 7.0}
    lat = {"heads": H, "dim": D, "rot_dim": D // 2, "vdim": D, "q_rank": 3 * d // 8, "kv_rank": 4 * D, "scale": (D + D // 2) ** -0.5,
           "rot": {"base": 10000.0, "dims": D // 2, "scaling": {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}}}
    ret = {"heads": H, "dim": D, "vdim": D, "decay": [1.0 - 2.0 ** (-4 - 4 * h / max(H - 1, 1)) for h in range(H)],
           "rot": {"base": 10000.0, "dims": D}}
    specs = []
    for i in range(layers):
        kind = pattern[i % len(pattern)]
        mlp = moe if (i // 2 + i) % 2 == 0 else dense
        specs.append({"type": "latent_attention", "mixer": lat, "mlp": mlp} if kind in "la" else
                     {"type": "retention", "mixer": ret, "mlp": mlp})
    cfg = LimatarConfig.from_dict({"architecture": "Limatar", "layers": specs, "norm": {"eps": 1e-6}, "vocab": size["vocab"],
                                   "width": d}, name="limatar-bench")
    return LimatarModel(cfg, device=device, seed=seed)


def _rerozen(size: dict, layers: int, device, seed: int, pattern: str = "p2", chunk: int = 1024):
    """Layers alternating (``pattern``: p / 2 per layer, repeated; a / d and l / r of the other designs' patterns mean the
    same) between "parallel" (attention with biases and q / k norms beside gated linear attention) and "parallel_2"
    (attention with short convolutions, rotated values and a sink beside the gated delta rule).  The attention has the
    other designs' heads and head size and chunks of ``chunk`` positions; the linear attention half as many heads of the
    same size; the ungated feed-forward's two matrices get 1.5x the gated designs' inner width (equal parameters)."""
    from llm_weighted_consensus_amd.models.config import RerozenConfig
    from llm_weighted_consensus_amd.models.rerozen import RerozenModel

    H, G, D, d = size["heads"], size["kv_heads"], size["head_dim"], size["width"]
    rot = {"base": 10000.0, "dims": D // 2, "scaling": {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}}
    left = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "mask": {"size": chunk}, "rot": rot}
    mlp = {"kind": "dense", "ff": 3 * size["ffn"] // 2}
    two = {"type": "parallel_2", "mlp": mlp,
           "mixer": {"left": dict(left, conv=4), "right": {"heads": H // 2, "kv_heads": max(G // 2, 1), "dim": D, "vdim": D, "conv": 4,
                                                           "a_rank": 64, "g_rank": 64},
                     "left_scale": 0.7, "right_scale": 1.1}}
    one = {"type": "parallel", "mlp": mlp,
           "mixer": {"left": left, "right": {"heads": H // 2, "dim": D, "vdim": D, "tau": 16.0, "a_rank": 64},
                     "left_scale": 1.2, "right_scale": 0.5}}
    kinds = {"p": one, "a": one, "l": one, "2": two, "d": two, "r": two}
    cfg = RerozenConfig.from_dict({"architecture": "Rerozen", "canon": {"taps": 4}, "embedding": {"scale": d ** 0.5},
                                   "layers": [kinds[pattern[i % len(pattern)]] for i in range(layers)], "logit_scale": 0.25,
                                   "norm": {"eps": 1e-6}, "vocab": size["vocab"], "width": d}, name="rerozen-bench")
    return RerozenModel(cfg, device=device, seed=seed)


def _mixtral(size: dict, layers: int, max_pos: int, device, seed: int, experts: int = 8, top: int = 2):
    from llm_weighted_consensus_amd.models.config import DecoderConfig
    from llm_weighted_consensus_amd.models.mixtral import MixtralModel

    cfg = DecoderConfig("mixtral-bench", size["vocab"], size["width"], layers, size["heads"], size["kv_heads"],
                        size["head_dim"], size["ffn"] // top, max_position=max_pos, num_experts=experts, experts_per_token=top)
    return MixtralModel(cfg, device=device, seed=seed, max_position=max_pos)


def _measure(model, prompt_len: int, n_prompts: int, batch: int, gen: int, reps: int) -> dict:
    import torch

    from llm_weighted_consensus_amd.engine.engine import LLMEngine
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams
    from llm_weighted_consensus_amd.engine.tokenizer import ByteTokenizer

    V = model.cfg.vocab_size
    bs = 16
    blocks = (max(n_prompts, batch) + 2) * (-(-(prompt_len + gen + 16) // bs) + 1)
    eng = LLMEngine(model, ByteTokenizer(V), num_blocks=blocks, max_batch=max(batch, n_prompts),
                    max_model_len=prompt_len + gen + 16, prefill_token_budget=n_prompts * prompt_len, prefix_sharing=False,
                    kv_reserve_tokens=None)
    g = torch.Generator().manual_seed(7)

    def prompts(n):
        return [torch.randint(0, 255, (prompt_len,), generator=g).tolist() for _ in range(n)]

    def run(n, new):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.generate(prompts(n), SamplingParams(temperature=0.0, max_tokens=new, ignore_eos=True))
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    run(n_prompts, 1)          # warm-up: kernels, library heuristics
    run(batch, gen)            # warm-up: the decode bucket's tuning and graph capture
    t_pre = min(run(n_prompts, 1) for _ in range(reps))
    t_one = min(run(batch, 1) for _ in range(reps))
    t_gen = min(run(batch, gen) for _ in range(reps))
    del eng
    torch.cuda.empty_cache()
    return {"prefill_tok_s": n_prompts * prompt_len / t_pre, "prefill_ms": t_pre * 1e3,
            "decode_tok_s": batch * (gen - 1) / max(t_gen - t_one, 1e-9), "decode_ms_per_step": (t_gen - t_one) / (gen - 1) * 1e3}


def run(sizes: str = "small,8b-layer", layers: int = 4, prompt_len: int = 2048, n_prompts: int = 8, batch: int = 64,
        gen: int = 33, window: int = 0, reps: int = 2, designs: str = "madipel,llama", pattern: str = "ad") -> int:
    import torch

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    window = window or (prompt_len + gen + 16)  # default: the window covers the context (equal attention work)
    summary = {}
    for name in sizes.split(","):
        size = SIZES[name]
        for design in designs.split(","):
            if design == "madipel":
                model = _madipel(size, layers, window, dev, 3)
            elif design == "merudra":
                model = _merudra(size, layers, dev, 3, pattern="".join({"l": "a", "r": "d", "p": "a", "2": "d"}.get(c, c) for c in pattern))
            elif design == "rerozen":
                model = _rerozen(size, layers, dev, 3, pattern=pattern)
            elif design == "limatar":
                model = _limatar(size, layers, dev, 3, pattern=pattern)
            elif design == "mixtral":
                model = _mixtral(size, layers, prompt_len + gen + 80, dev, 3)
            else:
                model = _llama(size, layers, prompt_len + gen + 80, dev, 3)
            r = _measure(model, prompt_len, n_prompts, batch, gen, reps)
            params = model.cfg.params()
            del model
            torch.cuda.empty_cache()
            line = {"bench": "compare-decoders", "size": name, "design": design, "layers": layers, "params": params,
                    "prompt_len": prompt_len, "prompts": n_prompts, "decode_batch": batch, "window": window if design == "madipel" else None,
                    **{k: round(v, 3) for k, v in r.items()}, "dtype": "bf16", "data": "synthetic"}
            print(json.dumps(line), flush=True)
            summary.setdefault(name, {})[design] = r
    for a, b in (("madipel", "llama"), ("merudra", "mixtral"), ("merudra", "madipel"), ("limatar", "merudra"), ("rerozen", "merudra")):
        out = {}
        for name, d in summary.items():
            if a in d and b in d:
                out[name] = {"prefill_ratio": round(d[a]["prefill_tok_s"] / d[b]["prefill_tok_s"], 3),
                             "decode_ratio": round(d[a]["decode_tok_s"] / d[b]["decode_tok_s"], 3)}
        if out:
            print(json.dumps({"bench": "compare-decoders", f"{a}_over_{b}": out}), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(run())
