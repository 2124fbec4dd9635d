"""Limatar on the CPU: config parsing, the order of layer runs, the registry, the rotation frequencies and the
plain oracle's own consistency (the GPU tests cover the kernels and the model)."""
import json
import math

import pytest
import torch

import limatar_oracle as O

SCALING = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
LAYERS = [O.retention_layer(2, 32, 16, O.dense(72, limit=2.5), rot_dims=16),
          O.latent_layer(4, 16, 8, 24, 20, 40, O.moe(8, 3, 24, shared=40), scale=0.21, scaling=SCALING),
          O.latent_layer(3, 10, 6, 14, 13, 27, O.moe(5, 1, 18)),
          O.retention_layer(3, 24, 40, None)]


def test_config_from_json_runs_and_registry(tmp_path):
    from llm_weighted_consensus_amd.models.config import (ClampedGluSpec, LimatarConfig, TopkExpertsSpec,
                                                          load_model_config)
    from llm_weighted_consensus_amd.models.registry import model_class

    cfg = O.make_config(40, 77, LAYERS, loop=(1, 3, 3), eps=1e-4)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    c = load_model_config(tmp_path)
    assert isinstance(c, LimatarConfig) and c.vocab_size == 77 and c.hidden == 40 and c.norm_eps == 1e-4
    assert c.runs == (0, 1, 2, 1, 2, 1, 2, 3) == tuple(O.layer_runs(cfg)) and c.layers == 8
    r, a, b, last = c.layer_specs
    assert (r.type, r.mixer.nq, r.mixer.nv, r.mixer.rot.dims, len(r.mixer.decay)) == ("retention", 64, 32, 16, 2)
    assert isinstance(r.mlp, ClampedGluSpec) and (r.mlp.ff, r.mlp.limit, r.mlp.alpha) == (72, 2.5, 1.702)
    assert (a.type, a.mixer.nq, a.mixer.nv, a.mixer.q_rank, a.mixer.kv_rank, a.mixer.scale) == ("latent_attention", 96, 96, 20, 40, 0.21)
    assert a.mixer.rot.scaling == (4.0, 64.0, 8.0, 1.0) and b.mixer.rot.scaling is None
    assert isinstance(a.mlp, TopkExpertsSpec) and (a.mlp.experts, a.mlp.top, a.mlp.ff, a.mlp.shared_ff) == (8, 3, 24, 40)
    assert b.mlp.shared_ff == 0 and last.mlp is None
    assert LimatarConfig.from_dict({**cfg, "loop": None}).runs == (0, 1, 2, 3)
    assert model_class(c).__name__ == "LimatarModel"
    assert c.params() == sum(t.numel() for t in O.make_weights(cfg, 0).values())
    for path, value in ((("layers", 1, "mixer", "rot", "dims"), 6), (("layers", 0, "mixer", "decay"), [0.5]),
                        (("layers", 0, "type"), "other"), (("layers", 1, "mlp", "kind"), "other"),
                        (("loop", "stop"), 9), (("layers", 2, "mlp", "router", "top"), 6)):
        bad = json.loads(json.dumps(cfg))
        node = bad
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = value
        with pytest.raises(ValueError):
            LimatarConfig.from_dict(bad)


@pytest.mark.parametrize("dims,base,scaling", [(16, 30000.0, None), (6, 100.0, SCALING), (2, 50.0, SCALING),
                                               (64, 5e5, {**SCALING, "factor": 2.5, "original": 1000})])
def test_rotation_frequencies_against_the_oracle_tables(dims, base, scaling):
    from llm_weighted_consensus_amd.ops.res32 import rope_frequencies

    f, m = rope_frequencies(dims, base, scaling, "cpu")
    assert f.dtype == torch.float32 and f.shape == (dims // 2,)
    pos = torch.tensor([0, 1, 7, 300])
    cos, sin = O.rope_tables({"dims": dims, "base": base, "scaling": scaling}, pos)
    a = pos.double()[:, None] * f.double()[None, :]
    assert (torch.cos(a) * m - cos).abs().max() < 2e-5 and (torch.sin(a) * m - sin).abs().max() < 2e-5
    if scaling:
        assert abs(m - (0.1 * math.log(scaling["factor"]) + 1)) < 1e-12
        plain, _ = rope_frequencies(dims, base, None, "cpu")
        assert float((plain / f).max()) <= scaling["factor"] * (1 + 1e-6) and float((plain / f).min()) >= 1 - 1e-6


def test_oracle_mechanisms_agree_with_their_definitions():
    """The oracle's own pieces: sink softmax rows sum to 1 - the sink's share; the retention scan equals the explicit
    double sum with decay powers; rotations keep lengths and compose by position differences."""
    g = torch.Generator().manual_seed(0)
    s = torch.randn(2, 5, 7, generator=g, dtype=torch.float64)
    sink = torch.tensor([0.3, -2.0], dtype=torch.float64)
    p = O.sink_softmax(s, sink)
    share = torch.exp(sink)[:, None] / (torch.exp(s).sum(-1) + torch.exp(sink)[:, None])
    assert (p.sum(-1) + share - 1).abs().max() < 1e-12
    T, H, D, Dv = 9, 2, 4, 3
    q, k, v = (torch.randn(T, H, n, generator=g, dtype=torch.float64) for n in (D, D, Dv))
    decay = [0.5, 0.9]
    o, S = O.retention_scan(q, k, v, decay)
    for h in range(H):
        for i in range(T):
            ref = sum(decay[h] ** (i - j) * float(q[i, h] @ k[j, h]) * v[j, h] for j in range(i + 1))
            assert (o[i, h] - ref).abs().max() < 1e-12
    o2, S2 = O.retention_scan(q[5:], k[5:], v[5:], decay, S=O.retention_scan(q[:5], k[:5], v[:5], decay)[1])
    assert (o2 - o[5:]).abs().max() < 1e-12 and (S2 - S).abs().max() < 1e-12
    rot = {"dims": 4, "base": 100.0}
    cos, sin = O.rope_tables(rot, torch.arange(T))
    for rotate in (O.rotate_interleaved, O.rotate_half):
        a, b = rotate(q, cos, sin), rotate(k, cos, sin)
        assert (a.norm(dim=-1) - q.norm(dim=-1)).abs().max() < 1e-12
        c4, s4 = O.rope_tables(rot, torch.tensor([4]))
        c0, s0 = O.rope_tables(rot, torch.tensor([0]))
        moved = float((rotate(q[6:7], c4, s4)[0, 0] * rotate(k[2:3], c0, s0)[0, 0]).sum())
        assert abs(moved - float((a[6, 0] * b[2, 0]).sum())) < 1e-9  # only the distance 6 - 2 matters
