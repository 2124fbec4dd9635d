"""Rerozen on the CPU: config parsing, the low-rank widths taken from a checkpoint's shapes, the registry, and the
oracle's own pieces against closed forms (the GPU tests cover the kernels and the model)."""
import json
import math

import pytest
import torch

import rerozen_oracle as O

YARN = dict(factor=4.0, original=64, fast=8.0, slow=2.0)
LAYERS = [dict(type="parallel_2", left=O.attention_left(4, 2, 12, 10, 7, 8, conv=2, scaling=YARN),
               right=dict(heads=4, kv_heads=2, dim=12, vdim=20, conv=3), ff=24, a_rank=6, g_rank=5),
          dict(type="parallel", left=O.attention_left(2, 1, 16, 24, 20, 16, base=5000.0), right=dict(heads=3, dim=8, vdim=6, tau=4.0),
               ff=None, left_scale=1.2, right_scale=0.4, a_rank=3)]


def test_config_from_json_ranks_and_registry(tmp_path):
    from llm_weighted_consensus_amd.models.config import RerozenConfig, load_model_config
    from llm_weighted_consensus_amd.models.registry import model_class

    cfg, ranks = O.make_config(40, 77, LAYERS, taps=3, embed_scale=6.5, logit_scale=0.3)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    c = load_model_config(tmp_path)
    assert isinstance(c, RerozenConfig) and c.layers == 2 and c.canon_taps == 3 and c.vocab_size == 77 and c.hidden == 40
    assert c.embed_scale == 6.5 and c.logit_scale == 0.3 and c.heads == 4 and c.kv_heads == 2 and c.head_dim == 16
    a, b = c.layer_specs
    assert (a.type, a.left.conv, a.left.sink, a.left.rotate_values, a.left.bias, a.left.qk_norm) == ("parallel_2", 2, True, True, False, False)
    assert (a.left.chunk, a.left.rot.dims, a.left.rot.scaling, a.left.nq, a.left.nk, a.left.nv) == (7, 8, (4.0, 64.0, 8.0, 2.0), 48, 24, 20)
    assert (a.right.kind, a.right.conv, a.right.nq, a.right.nv, a.right.nd, a.ff) == ("delta", 3, 24, 80, 48, 24)
    assert (b.type, b.left.conv, b.left.sink, b.left.bias, b.left.qk_norm, b.left.rot.scaling) == ("parallel", 0, False, True, True, None)
    assert (b.right.kind, b.right.kv_heads, b.right.tau, b.left_scale, b.right_scale, b.ff) == ("gla", 3, 4.0, 1.2, 0.4, 0)
    assert a.right.a_rank == 0 and a.right.g_rank == 0          # the config leaves them to the checkpoint
    W = O.make_weights(cfg, ranks, 0)
    full = c.with_ranks({k: tuple(v.shape) for k, v in W.items()})
    assert (full.layer_specs[0].right.a_rank, full.layer_specs[0].right.g_rank, full.layer_specs[1].right.a_rank) == (6, 5, 3)
    assert full.params() == sum(t.numel() for t in W.values())
    assert model_class(c).__name__ == "RerozenModel"
    for edit in (lambda x: x["layers"][0].__setitem__("type", "other"),
                 lambda x: x["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3),
                 lambda x: x["layers"][1]["mixer"]["left"]["rot"].__setitem__("dims", 18),
                 lambda x: x["layers"][0]["mixer"]["left"]["mask"].__setitem__("size", 0),
                 lambda x: x["layers"][1].__setitem__("mlp", dict(kind="moe", ff=8))):
        bad = json.loads(json.dumps(cfg))
        edit(bad)
        with pytest.raises(ValueError):
            RerozenConfig.from_dict(bad)


def test_oracle_pieces_against_closed_forms():
    """The oracle's masks, rotation and recurrences on inputs whose answers are known."""
    m = O.chunk_mask(7, 3)
    assert m.int().tolist() == [[1, 0, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0, 0], [0, 0, 0, 1, 0, 0, 0],
                                [0, 0, 0, 1, 1, 0, 0], [0, 0, 0, 1, 1, 1, 0], [0, 0, 0, 0, 0, 0, 1]]
    # a rotation keeps lengths and turns back; without scaling the first pair turns by one radian per position
    x = torch.randn(5, 2, 10, dtype=torch.float64)
    f, mult = O.rope_freqs(6, 100.0)
    pos = torch.arange(5)
    y = O.rotate(x, pos, f, mult)
    assert mult == 1.0 and float(f[0]) == 1.0 and torch.equal(y[..., 6:], x[..., 6:])
    assert (y.norm(dim=-1) - x.norm(dim=-1)).abs().max() < 1e-12 and (O.rotate(y, pos, f, sign=-1.0) - x).abs().max() < 1e-12
    assert abs(float(y[1, 0, 0]) - (float(x[1, 0, 0]) * math.cos(1) - float(x[1, 0, 3]) * math.sin(1))) < 1e-12
    fs, ms = O.rope_freqs(8, 10000.0, dict(factor=4.0, original=64, fast=8.0, slow=2.0))
    assert abs(ms - (0.1 * math.log(4.0) + 1)) < 1e-15 and float(fs[0]) == 1.0 and abs(float(fs[3]) - 10000.0 ** -0.75 / 4) < 1e-15
    # the softmax with a sink: uniform scores over n keys give weights 1 / (n + 1)
    q, k, v = torch.zeros(4, 1, 2, dtype=torch.float64), torch.zeros(4, 1, 2, dtype=torch.float64), torch.ones(4, 1, 3, dtype=torch.float64)
    o = O.chunked_softmax_attention(q, k, v, 1.0, 3, sink=True)
    assert (o[:, 0, 0] - torch.tensor([1 / 2, 2 / 3, 3 / 4, 1 / 2], dtype=torch.float64)).abs().max() < 1e-12
    # delta rule with beta = 1 and no decay stores v under k exactly; a second write under the same key replaces it
    k = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]]], dtype=torch.float64)
    v = torch.tensor([[[2.0, 3.0]], [[5.0, 7.0]]], dtype=torch.float64)
    one = torch.ones(2, 1, 2, dtype=torch.float64)
    o, S = O.recurrence(k, k, v, one, torch.ones(2, 1, dtype=torch.float64))
    assert torch.equal(o[1, 0], v[1, 0]) and torch.equal(S[0, 0], v[1, 0])
    o, S = O.recurrence(k, k, v, one * 0.5)                      # plain accumulation: 0.5 * first + second
    assert torch.equal(o[1, 0], 0.5 * v[0, 0] + v[1, 0])
    assert (O.causal_conv(torch.arange(4.0).view(4, 1), torch.tensor([[1.0, 10.0, 100.0]])).flatten() - torch.tensor([0.0, 100.0, 210.0, 321.0])).abs().max() == 0
