"""Limatar on the GPU against the plain fp64 oracle (tests/limatar_oracle.py): each mechanism alone, then the model
through the engine — whole prompts, token-by-token decoding, portions, unequal batches, pages and state slots used
again, the first tokens of a sequence, keys far away and at page borders, long decoding, the looped span and greedy
generation through the scheduler.  Small configurations with random weights; sizes chosen so that nothing the design
allows to differ happens to be equal or 1."""
import json
import math

import pytest
import torch

import limatar_oracle as O

pytestmark = pytest.mark.gpu

F64 = torch.float64
SCALING = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def _items(lens, slots, starts, gpu):
    """StepItems of portions with ``lens`` rows starting at positions ``starts`` in state slots ``slots``."""
    from llm_weighted_consensus_amd.ops import res32

    cu, row_item, pos = [0], [], []
    for i, (n, p0) in enumerate(zip(lens, starts)):
        cu.append(cu[-1] + n)
        row_item += [i] * n
        pos += list(range(p0, p0 + n))
    t = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)  # noqa: E731
    return res32.StepItems(t(row_item), t(cu), t(slots), t(pos))


# ------------------------------------------------------------------ mechanisms, one by one
@pytest.mark.parametrize("dims,base,scaling", [(16, 30000.0, None), (6, 100.0, SCALING), (64, 5e5, {**SCALING, "factor": 2.5, "original": 1000})])
def test_rotation_frequencies(gpu, dims, base, scaling):
    from llm_weighted_consensus_amd.ops import res32

    f, m = res32.rope_frequencies(dims, base, scaling, gpu)
    pos = torch.tensor([0, 1, 7, 300])
    cos, sin = O.rope_tables({"dims": dims, "base": base, "scaling": scaling}, pos)
    a = pos.double()[:, None] * f.cpu().double()[None, :]
    assert (torch.cos(a) * m - cos).abs().max() < 2e-5 and (torch.sin(a) * m - sin).abs().max() < 2e-5
    if scaling:
        assert abs(m - (0.1 * math.log(scaling["factor"]) + 1)) < 1e-12
        plain, _ = res32.rope_frequencies(dims, base, None, gpu)
        assert float((plain / f).max()) > 1.5  # the slow pairs were stretched


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("H,D,R,C,Cq", [(3, 20, 6, 28, 12), (2, 32, 16, 104, 72), (5, 8, 2, 5, 7)])
def test_latent_cache_rows_and_query_rows(gpu, dtype, tol, H, D, R, C, Cq):
    """From projected rows to what the attention reads: the normalised query latent, the cached key row [latent |
    rotated part | zeros], the latent again in the interleaved value row, and the fp32 query rows [absorbed part |
    rotated part | zeros] — positions far from zero, slots scattered over pages."""
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(H + C)
    T, bs, eps, scale = 11, 8, 1e-5, 0.37
    Dk, Cv = -(-(C + R) // 8) * 8, -(-C // 8) * 8
    rot = {"dims": R, "base": 777.0, "scaling": SCALING}
    proj = torch.randn(T, Cq + C + R + 5, generator=g).to(dtype)
    wq, wc = 1 + 0.2 * torch.randn(Cq, generator=g), 1 + 0.2 * torch.randn(C, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 50, 51, 52, 997, 998, 999, 1000], dtype=torch.int32)
    slots = torch.randperm(4 * bs, generator=g)[:T].to(torch.int32)
    cache = PagedLayerCache([(Dk, Cv)], 4, bs, gpu, dtype)
    cache.pool.fill_(7.0)  # stale contents
    f, m = res32.rope_frequencies(R, rot["base"], rot["scaling"], gpu)
    cq = res32.latent_kv_write(proj.to(gpu), Cq, C, R, wq.to(gpu), wc.to(gpu), f, m, pos.to(gpu), slots.to(gpu), cache.k[0],
                               cache.v[0], eps)
    p64 = proj.double()
    cos, sin = O.rope_tables(rot, pos)
    ref_cq = O.norm_plain(p64[:, :Cq], wq, eps)
    ref_c = O.norm_plain(p64[:, Cq:Cq + C], wc, eps)
    ref_kr = O.rotate_interleaved(p64[:, Cq + C:Cq + C + R], cos, sin)
    krow, vrow = cache.rows(0, slots.long().to(gpu))
    assert (cq.cpu().double() - ref_cq).abs().max() < tol * 4
    assert (krow[:, :C].cpu().double() - ref_c).abs().max() < tol * 4
    assert (krow[:, C:C + R].cpu().double() - ref_kr).abs().max() < tol * 4
    assert (vrow[:, :C].cpu().double() - ref_c).abs().max() < tol * 4
    assert float(krow[:, C + R:].abs().sum()) == 0 and float(vrow[:, C:].abs().sum()) == 0
    q = torch.randn(T, H * (D + R), generator=g).to(dtype)
    qn = torch.randn(H, T, C, generator=g)
    qf = res32.latent_q_rows(q.to(gpu), D, R, qn.to(gpu), f, m, scale, pos.to(gpu), H, Dk).cpu().double()
    ref_rot = O.rotate_interleaved(q.double().view(T, H, D + R)[..., D:], cos, sin) * scale
    assert (qf[..., :C] - qn.double().transpose(0, 1) * scale).abs().max() < 1e-5
    assert (qf[..., C:C + R] - ref_rot).abs().max() < 2e-5 * max(1.0, float(ref_rot.abs().max()))
    assert float(qf[..., C + R:].abs().sum()) == 0
    # without the absorbed part: the rows' own unrotated entries (attention over up-projected keys)
    Dq = -(-(D + R) // 32) * 32
    q2 = res32.latent_q_rows(q.to(gpu), D, R, None, f, m, scale, pos.to(gpu), H, Dq).cpu().double()
    assert (q2[..., :D] - q.double().view(T, H, D + R)[..., :D] * scale).abs().max() < 1e-5
    assert (q2[..., D:D + R] - ref_rot).abs().max() < 2e-5 * max(1.0, float(ref_rot.abs().max()))
    assert float(q2[..., D + R:].abs().sum()) == 0


@pytest.mark.parametrize("d", [44, 64, 1028, 4096])
def test_residual_add_with_both_norms_in_one_pass(gpu, d):
    """x += norm(y) (1 + w) and, in the same pass, the next sublayer's input norm of the new x (bf16 rows), against the
    oracle; the plain row norm (fp32 and bf16 rows, gathered rows) beside it."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(d)
    T, eps = 9, 1e-5
    x, y = torch.randn(T, d, generator=g) * 3, torch.randn(T, d, generator=g).to(torch.bfloat16)
    w, wn = 0.1 * torch.randn(d, generator=g), 0.1 * torch.randn(d, generator=g)
    ref_x = x.double() + O.norm_zero_centered(y.double(), w, eps)
    ref_h = O.norm_zero_centered(ref_x, wn, eps)
    xg, h = x.to(gpu), torch.empty(T, d, dtype=torch.bfloat16, device=gpu)
    res32.gated_norm_residual(xg, y.to(gpu), (1 + w).to(gpu), eps, x_cast=h, next_w=(1 + wn).to(gpu))
    assert (xg.cpu().double() - ref_x).abs().max() < 1e-5 * 8
    assert (h.cpu().double() - ref_h).abs().max() < 3e-2
    rows = torch.tensor([4, 0, 8])
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        got = res32.rmsnorm_rows(xg, (1 + wn).to(gpu), eps, dt).cpu().double()
        assert (got - ref_h).abs().max() < tol * 4
        got = res32.rmsnorm_rows(xg, (1 + wn).to(gpu), eps, dt, rows=rows.to(gpu)).cpu().double()
        assert (got - ref_h[rows]).abs().max() < tol * 4


def _paged(n_tokens, bs, nk, nv, dtype, gpu, seed=0):
    """A cache of shuffled pages for one sequence of n_tokens: (cache, table row, slots)."""
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache

    nb = -(-n_tokens // bs)
    perm = torch.randperm(nb + 3, generator=torch.Generator().manual_seed(seed))[:nb]
    cache = PagedLayerCache([(nk, nv)], nb + 3, bs, gpu, dtype)
    slots = torch.tensor([int(perm[j // bs]) * bs + j % bs for j in range(n_tokens)])
    return cache, perm.to(torch.int32), slots


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,D,Dv", [(3, 40, 24), (7, 120, 88), (2, 328, 320), (1, 8, 8), (4, 128, 128), (5, 64, 32), (20, 64, 32), (3, 192, 128),
                                    (17, 576, 512)])
def test_softmax_with_sinks_over_one_shared_row(gpu, dtype, tol, H, D, Dv):
    """All heads read ONE cached row per token (G = 1); exp(sink_h) joins the denominator.  Decode rows and a prompt
    portion behind a cached head, sinks from far below to far above the scores.  In bf16 the sizes the matrix-core
    kernels are built for run there (decode rows split over the keys; 17 heads: two head chunks), the rest and fp32 on
    the general kernel."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(D)
    n, bs = 83, 16
    cache, table, slots = _paged(n, bs, D, Dv, dtype, gpu, seed=D)
    K, V = torch.randn(n, D, generator=g).to(dtype), torch.randn(n, Dv, generator=g).to(dtype)
    latent = D == 576  # the wide decode kernel reads its values from the key rows: the values are the rows' head
    if latent:
        V = K[:, :Dv].clone()
    cache.set_rows(0, slots.to(gpu), K.to(gpu), V.to(gpu))
    sink = torch.linspace(-30.0, 6.0, H) if H > 1 else torch.tensor([1.5])
    q = torch.randn(n, H, D, generator=g) * D ** -0.5
    s = torch.einsum("ihd,jd->hij", q.double(), K.double())
    pos = torch.arange(n)
    s = s.masked_fill(pos[None, :, None] < pos[None, None, :], -math.inf)
    ref = torch.einsum("hij,jv->ihv", O.sink_softmax(s, sink.double()), V.double())
    z = torch.zeros(H, device=gpu)
    tab = table[None].to(gpu)
    rows = [0, 1, 15, 16, 17, 82]  # decode rows: every row its own item
    out = torch.empty(len(rows), H * Dv, dtype=dtype, device=gpu)
    res32.window_attn(q[rows].reshape(len(rows), -1).to(gpu), cache.k[0], cache.v[0], torch.tensor(rows, dtype=torch.int32, device=gpu),
                      tab.expand(len(rows), -1).contiguous(), z, z, 1 << 30, out, H, 1, sink=sink.to(gpu), cores=True,
                      values_in_keys=latent)
    assert (out.cpu().double().view(len(rows), H, Dv) - ref[rows]).abs().max() < tol * 4
    a = 30  # a portion of rows a .. n-1 behind a cached head
    out = torch.empty(n - a, H * Dv, dtype=dtype, device=gpu)
    res32.window_attn(q[a:].reshape(n - a, -1).to(gpu), cache.k[0], cache.v[0], torch.arange(a, n, dtype=torch.int32, device=gpu), tab, z, z,
                      1 << 30, out, H, 1, cu_q=torch.tensor([0, n - a], dtype=torch.int32, device=gpu),
                      k_lens=torch.tensor([n], dtype=torch.int32, device=gpu), max_q=n - a, sink=sink.to(gpu), cores=True)
    assert (out.cpu().double().view(n - a, H, Dv) - ref[a:]).abs().max() < tol * 4
    if H > 1:  # the lowest sink changes nothing, the highest takes most of the weight
        w = O.sink_softmax(s, sink.double())[:, -1].sum(-1)
        assert abs(float(w[0]) - 1) < 1e-9 and float(w[-1]) < 0.5


@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dtype,D,Dv", [(torch.float32, 24, 16), (torch.bfloat16, 24, 16), (torch.bfloat16, 128, 64)])
def test_far_key_and_page_borders_stand_out(gpu, decode, dtype, D, Dv):
    """One key made to stand out (its row parallel to the query, scaled up) at the first token, at both sides of page
    borders and hundreds of tokens back over shuffled pages: the result is that key's value row, less the sink's share."""
    from llm_weighted_consensus_amd.ops import res32

    H, n, bs = 2, 300, 16
    g = torch.Generator().manual_seed(5)
    z = torch.zeros(H, device=gpu)
    sink = torch.tensor([-50.0, 2.0])
    for target in (0, 15, 16, 17, 31, 32, 298, 299):
        cache, table, slots = _paged(n, bs, D, Dv, dtype, gpu, seed=target)
        K, V = 0.05 * torch.randn(n, D, generator=g), torch.randn(n, Dv, generator=g)
        qv = torch.randn(D, generator=g)
        qv = qv / qv.norm()
        K[target] = 12.0 * qv
        cache.set_rows(0, slots.to(gpu), K.to(dtype).to(gpu), V.to(dtype).to(gpu))
        q = (qv[None, None] * 3.0).expand(1, H, D).reshape(1, H * D).contiguous().to(gpu)
        out = torch.empty(1, H * Dv, dtype=dtype, device=gpu)
        kw = {} if decode else dict(cu_q=torch.tensor([0, 1], dtype=torch.int32, device=gpu),
                                    k_lens=torch.tensor([n], dtype=torch.int32, device=gpu), max_q=1)
        res32.window_attn(q, cache.k[0], cache.v[0], torch.tensor([n - 1], dtype=torch.int32, device=gpu), table[None].to(gpu), z, z,
                          1 << 30, out, H, 1, sink=sink.to(gpu), cores=True, **kw)
        got = out.cpu().double().view(H, Dv)
        want = V[target].to(dtype).double()
        assert (got[0] - want).abs().max() < 2e-2, target                       # no sink to speak of
        share = 1.0 / (1.0 + math.exp(2.0 - 36.0))
        assert (got[1] - want * share).abs().max() < 2e-2, target


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,D,Dv,rd", [(3, 12, 20, 8), (2, 64, 64, 64), (4, 64, 48, 64), (2, 80, 72, 40), (1, 130, 8, 0), (2, 200, 40, 200)])
def test_retention_portions_single_tokens_and_stale_slots(gpu, dtype, tol, H, D, Dv, rd):
    """The recurrence with its rotation: two sequences cut into portions (single rows, two tokens, the two interleaved
    in one step, tiles of the kernel crossed) in slots that held other data, against the whole-sequence oracle; the
    state left in the slot is the oracle's."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(D + Dv)
    na, nb = 61, 9
    decay = [1.0 - 2.0 ** (-1 - 2 * h) for h in range(H)]
    rot = {"dims": rd, "base": 500.0}
    f, m = res32.rope_frequencies(rd, rot["base"], None, gpu)
    nq, nv = H * D, H * Dv
    width = 2 * nq + nv + 3
    seqs = {"a": torch.randn(na, width, generator=g).to(dtype), "b": torch.randn(nb, width, generator=g).to(dtype)}
    state = (torch.randn(4, H, D, Dv, generator=g) * 50).to(gpu)  # stale contents of earlier sequences
    ref, ref_S = {}, {}
    for k, x in seqs.items():
        T = x.shape[0]
        x64 = x.double()
        q, kk = x64[:, :nq].reshape(T, H, D).clone(), x64[:, nq:2 * nq].reshape(T, H, D).clone()
        if rd:
            cos, sin = O.rope_tables(rot, torch.arange(T))
            q[..., :rd], kk[..., :rd] = O.rotate_half(q[..., :rd], cos, sin), O.rotate_half(kk[..., :rd], cos, sin)
        ref[k], ref_S[k] = O.retention_scan(q, kk * D ** -0.5, x64[:, 2 * nq:2 * nq + nv].reshape(T, H, Dv), decay)
    plan = [[("a", 1)], [("a", 2), ("b", 1)], [("b", 2), ("a", 1)], [("a", 17)], [("b", 6), ("a", 33)], [("a", 7)]]
    at, got, slot = {"a": 0, "b": 0}, {"a": [], "b": []}, {"a": 2, "b": 0}
    dec = torch.tensor(decay, dtype=torch.float32, device=gpu)
    for step in plan:
        x = torch.cat([seqs[k][at[k]:at[k] + n] for k, n in step]).to(gpu)
        items = _items([n for _, n in step], [slot[k] for k, _ in step], [at[k] for k, _ in step], gpu)
        out = res32.retention(x, nq, x[:, 2 * nq:2 * nq + nv], f, m, rd, dec, state, items, H)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n].cpu())
            o, at[k] = o + n, at[k] + n
    assert at == {"a": na, "b": nb}
    for k in seqs:
        r = ref[k].reshape(-1, nv)
        assert (torch.cat(got[k]).double() - r).abs().max() < tol * 4 * max(1.0, float(r.abs().max())), k
        assert (state[slot[k]].cpu().double() - ref_S[k]).abs().max() < tol * 4 * max(1.0, float(ref_S[k].abs().max())), k


def test_retention_far_token_survives_a_slow_decay(gpu):
    """One early token made large: after hundreds of tokens its share of the result is a^n times its value, for a fast
    and a slow head (prompt portion, then single tokens)."""
    from llm_weighted_consensus_amd.ops import res32

    H, D, Dv, n = 2, 16, 16, 400
    decay = [0.9, 0.9990234375]
    g = torch.Generator().manual_seed(3)
    x = 0.01 * torch.randn(n, 2 * H * D + H * Dv, generator=g)
    unit = torch.zeros(D)
    unit[3] = 1.0
    x[5, :H * D] = 0
    x[5, H * D:2 * H * D] = (unit * 100.0 * D ** 0.5).repeat(H)   # k of token 5
    x[5, 2 * H * D:] = 1.0                                         # v of token 5
    x[n - 1, :H * D] = unit.repeat(H)                              # q of the last token
    f, m = res32.rope_frequencies(0, 10.0, None, gpu)
    dec = torch.tensor(decay, device=gpu)
    for cut in (n, n - 20):
        state = torch.zeros(2, H, D, Dv, device=gpu)
        xs = x.to(gpu)
        outs = [res32.retention(xs[:cut], H * D, xs[:cut, 2 * H * D:], f, m, 0, dec, state, _items([cut], [1], [0], gpu), H)]
        for t in range(cut, n):
            outs.append(res32.retention(xs[t:t + 1], H * D, xs[t:t + 1, 2 * H * D:], f, m, 0, dec, state, _items([1], [1], [t], gpu), H))
        last = torch.cat(outs)[-1].cpu().view(H, Dv)
        for h in range(H):
            want = 100.0 * decay[h] ** (n - 1 - 5)
            assert abs(float(last[h].mean()) - want) < 0.02 + 1e-3 * want, (cut, h)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("n", [7, 64, 96])
def test_gated_units(gpu, dtype, tol, n):
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(n)
    gu = (3 * torch.randn(13, 2 * n + 4, generator=g)).to(dtype)
    x = gu.to(gpu)[:, :2 * n]
    a, b = gu.double()[:, :n], gu.double()[:, n:2 * n]
    for limit in (0.75, 7.0):
        got = res32.glu(x, mode="clamped", alpha=1.702, limit=limit).cpu().double()
        assert (got - O.clamped_unit(a, b, limit)).abs().max() < tol * 8
    got = res32.glu(x).cpu().double()
    assert (got - a * torch.sigmoid(a) * b).abs().max() < tol * 30


@pytest.mark.parametrize("E,top,d", [(5, 3, 24), (16, 1, 24), (40, 4, 23), (90, 6, 16)])
def test_router_largest_logits_softmax_over_the_chosen(gpu, E, top, d):
    """Choice by the logits + bias, weights = softmax over the chosen logits only; the expert-major row lists are
    consistent; the combine adds a shared expert's rows."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(E)
    T = 37
    h = torch.randn(T, d, generator=g)
    Wr, b = torch.randn(E, d, generator=g), torch.randn(E, generator=g)
    z = (h @ Wr.T).to(gpu)
    ids, w, row_off, src, row_expert, inv = res32.router(z, None, E, top, bias=b.to(gpu), renorm=True)
    ref_ids, ref_w = O.route(h.double(), lambda n: {"router": Wr, "router.b": b}[n].double(), {"router": {"top": top}})
    assert torch.equal(ids.cpu().long(), ref_ids)
    assert (w.cpu().double() - ref_w).abs().max() < 1e-5 and (w.sum(-1) - 1).abs().max() < 1e-5
    assert int(row_off[-1]) == T * top
    rows = inv.cpu().view(T, top)
    assert torch.equal(src.cpu()[rows.flatten().long()].view(T, top), torch.arange(T)[:, None].expand(T, top).int())
    assert torch.equal(row_expert.cpu()[rows.flatten().long()].view(T, top), ids.cpu())
    Y = torch.randn(T * top, d, generator=g).to(gpu)
    add = torch.randn(T, d + 4, generator=g).to(gpu)[:, :d]
    got = res32.moe_combine(Y, inv, w, h.to(gpu), add=add).cpu().double()
    ref = (Y.cpu().double()[rows.long()] * ref_w[..., None]).sum(1) + add.cpu().double()
    assert (got - ref).abs().max() < 1e-4


# ------------------------------------------------------------------ the model through the engine
def _configs():
    m8 = O.moe(8, 3, 24, shared=40)
    out = {
        # both mixers, both feed-forwards, a looped span in the middle (three passes), a layer without feed-forward
        "mixed": dict(width=64, vocab=250, loop=(1, 3, 3), layers=[
            O.retention_layer(2, 32, 16, O.dense(72), rot_dims=16),
            O.latent_layer(4, 16, 8, 24, 20, 40, m8, scale=0.21, scaling=SCALING),
            O.retention_layer(3, 24, 40, None),
            O.latent_layer(2, 24, 16, 16, 48, 24, O.dense(96, limit=6.0))]),
        # odd sizes everywhere: nothing a multiple of 8, one head, one expert chosen, no shared expert, no loop
        "odd": dict(width=44, vocab=131, loop=None, layers=[
            O.latent_layer(3, 10, 6, 14, 13, 27, O.moe(5, 1, 18), scale=0.3),
            O.retention_layer(1, 20, 12, O.dense(50, limit=0.8), rot_dims=20),
            O.latent_layer(1, 12, 2, 6, 9, 11, None, scaling={**SCALING, "factor": 1.5})]),
        # retention only (no paged keys at all), the whole model looped twice
        "recurrent": dict(width=48, vocab=200, loop=(0, 2, 2), layers=[
            O.retention_layer(2, 64, 32, O.dense(64)), O.retention_layer(4, 16, 24, O.moe(4, 2, 16, shared=16), rot_dims=8)]),
        # attention only (no recurrent state), sizes of a matrix-core path (latent 96 + 32, values 96)
        "attentive": dict(width=64, vocab=200, loop=(1, 2, 2), layers=[
            O.latent_layer(4, 32, 32, 32, 32, 96, O.dense(64)), O.latent_layer(8, 16, 32, 16, 24, 96, m8, scaling=SCALING)]),
        # experts past the grouped-GEMM threshold
        "grouped": dict(width=256, vocab=200, loop=None, layers=[
            O.retention_layer(2, 32, 32, O.moe(4, 2, 1024, shared=64)), O.latent_layer(2, 32, 16, 32, 32, 48, O.dense(64))]),
    }
    # cached rows too wide for the portion kernel: prompt portions attend over up-projected keys and values (key sizes
    # 48 + 16 and 100 + 32 -> 192, values padded 40 -> 64), decode rows over the latent rows on the general kernel
    out["wide"] = dict(width=64, vocab=200, loop=(0, 1, 2), layers=[
        O.latent_layer(3, 48, 16, 32, 40, 200, O.dense(64)), O.latent_layer(2, 100, 32, 40, 24, 136, m8, scaling=SCALING)])
    # a latent wide enough for the 576 / 512 decode kernel (17 heads: two head chunks)
    out["deep"] = dict(width=64, vocab=200, loop=None, layers=[
        O.latent_layer(17, 16, 64, 16, 24, 320, O.dense(64)), O.retention_layer(2, 16, 16, None)])
    # a width that is no multiple of four (the kernels' one-element paths), 20 heads (two head chunks of the decode kernel),
    # 33 router outputs (the wave-wide router), a retention head wider than 128, the whole model looped
    out["ragged"] = dict(width=50, vocab=97, loop=(0, 2, 2), layers=[
        O.latent_layer(20, 6, 4, 5, 11, 26, O.moe(33, 4, 10)), O.retention_layer(2, 136, 20, O.dense(30, limit=2.0), rot_dims=100)])
    # the same layers with two passes of the span: bf16 comparisons (rounding differences grow with every pass of the
    # same weights, and a routing choice flipped by rounding changes a whole row)
    out["mixed2"] = {**out["mixed"], "loop": (1, 3, 2)}
    return out


CONFIGS = _configs()


def _make(name, seed=0):
    c = CONFIGS[name]
    cfg = O.make_config(c["width"], c["vocab"], c["layers"], loop=c["loop"])
    return cfg, O.make_weights(cfg, seed)


def _save(tmp_path, cfg, W):
    from safetensors.torch import save_file

    tmp_path.mkdir(exist_ok=True)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    return str(tmp_path)


def _build(tmp_path, name, dtype, seed=0, **engine_kw):
    from llm_weighted_consensus_amd.engine.engine import LLMEngine
    from llm_weighted_consensus_amd.engine.tokenizer import load_tokenizer
    from llm_weighted_consensus_amd.models.registry import load_model

    cfg, W = _make(name, seed)
    model = load_model(_save(tmp_path / f"{name}-{seed}", cfg, W), dtype=dtype)
    kw = dict(block_size=16, num_blocks=24, max_batch=4, max_model_len=256, use_graphs=False, prefix_sharing=False,
              tune_gc=False)
    kw.update(engine_kw)
    return cfg, W, model, LLMEngine(model, load_tokenizer({}, cfg["vocab"]), **kw)


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _err(got, ref, dtype=torch.float32):
    """fp32: the largest difference relative to the reference's largest entry (at least 1).  bf16: the row-wise relative RMS difference that 90 % of the rows stay under,
    times 4 (a routing choice that rounding flips changes single rows; that is not what is tested), and no row may be
    off by more than its own size."""
    d, ref = got.cpu().double() - ref, ref.double()
    if dtype == torch.float32:
        return float(d.abs().max()) / max(1.0, float(ref.abs().max()))
    rel = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert float(rel.max()) < 1.0
    return 4 * float(rel.flatten().quantile(0.9))


TOL = {torch.float32: 3e-4, torch.bfloat16: 0.5}


@pytest.mark.parametrize("name,dtype", [(n, d) for d in (torch.float32, torch.bfloat16) for n in ("mixed", "odd", "recurrent", "attentive", "wide", "deep", "ragged")
                                        if (n, d) != ("mixed", torch.bfloat16)] + [("mixed2", torch.bfloat16)])
def test_whole_prompt_and_layer_runs(gpu, tmp_path, name, dtype):
    """A whole prompt in one step: the stream after every layer RUN (looped layers count each time) and the logits."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(70, cfg["vocab"], 1)
    runs_ref, seen = [], []
    ref = O.forward(cfg, W, toks, runs_ref)
    model.on_layer = lambda ri, x: seen.append(x.detach().cpu().double())
    got = eng.step_tokens([("w", toks, list(range(len(toks))))], ["w"])
    model.on_layer = None
    assert len(seen) == len(runs_ref) == len(O.layer_runs(cfg))
    for a, b in zip(seen, runs_ref):
        assert _err(a, b, dtype) < TOL[dtype]
    assert _err(got, ref, dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


def test_grouped_expert_path(gpu, tmp_path):
    """Experts past the size threshold run through the framework's grouped GEMMs (bf16): a portion and single tokens."""
    from llm_weighted_consensus_amd import ops

    assert ops.available()
    cfg, W, model, eng = _build(tmp_path, "grouped", torch.bfloat16)
    assert cfg["width"] * cfg["layers"][0]["mlp"]["expert"]["ff"] >= model.GROUPED_MIN
    toks = _tokens(48, cfg["vocab"], 3)
    ref = O.forward(cfg, W, toks)
    got = [eng.step_tokens([("g", toks[:40], list(range(40)))])]
    for i in range(40, 48):
        got.append(eng.step_tokens([("g", [toks[i]], [0])], ["g"] if i == 47 else []))
    assert _err(torch.cat(got), ref, torch.bfloat16) < TOL[torch.bfloat16]


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("odd", torch.float32), ("attentive", torch.float32)])
def test_few_wanted_rows_and_what_they_leave(gpu, tmp_path, name, dtype):
    """A prompt of which only the last row is wanted (the last run's output side then runs on that row only): the same
    logits, and the cache and state it leaves carry the decoding that follows."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(60, cfg["vocab"], 6)
    ref = O.forward(cfg, W, toks)
    got = [eng.step_tokens([("k", toks[:50], [49])])]
    for i in range(50, 60):
        got.append(eng.step_tokens([("k", [toks[i]], [0])], ["k"] if i == 59 else []))
    assert _err(torch.cat(got), ref[49:], dtype) < TOL[dtype]


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("odd", torch.float32), ("recurrent", torch.float32),
                                        ("attentive", torch.bfloat16), ("mixed2", torch.bfloat16), ("wide", torch.bfloat16),
                                        ("deep", torch.bfloat16), ("ragged", torch.float32), ("ragged", torch.bfloat16)])
def test_decode_token_by_token_and_portions(gpu, tmp_path, name, dtype):
    """The same logits whether a prompt comes whole, token by token from the first token on, or in portions of
    changing sizes (down to two tokens; cut inside pages and inside the recurrence kernel's tiles)."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(75, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    rows = []
    for i, t in enumerate(toks):
        rows.append(eng.step_tokens([("d", [t], [0])], ["d"] if i + 1 == len(toks) else []))
    assert _err(torch.cat(rows), ref, dtype) < TOL[dtype]
    for sizes in ([2, 2, 13, 3, 16, 2, 30, 7], [17, 16, 15, 2, 25], [1, 2, 5, 67]):
        assert sum(sizes) == len(toks)
        rows, a = [], 0
        for n in sizes:
            rows.append(eng.step_tokens([("p", toks[a:a + n], list(range(n)))], ["p"] if a + n == len(toks) else []))
            a += n
        assert _err(torch.cat(rows), ref, dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("mixed2", torch.bfloat16), ("attentive", torch.bfloat16),
                                        ("odd", torch.float32), ("wide", torch.bfloat16), ("deep", torch.bfloat16)])
def test_unequal_batches_pages_and_slots_used_again(gpu, tmp_path, name, dtype):
    """Up to four live sequences of unequal lengths, portions beside single tokens, one sitting steps out, in a pool
    so small that pages and state slots are freed and taken again; every position equals the sequence run alone."""
    cfg, W, model, eng = _build(tmp_path, name, dtype, num_blocks=14)
    seqs = {k: _tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate([("a", 70), ("b", 12), ("c", 40), ("d", 33), ("e", 58), ("f", 1)])}
    ref = {k: O.forward(cfg, W, t) for k, t in seqs.items()}
    at = {k: 0 for k in seqs}
    plan = [[("a", 30), ("b", 2)], [("a", 1), ("b", 7), ("c", 17)], [("a", 1), ("c", 1), ("d", 33), ("b", 3)], [("a", 2), ("c", 22)],
            [("a", 36)], [("e", 20), ("f", 1)], [("e", 1)], [("e", 37)]]
    gots, refs, used = [], [], set()
    for step in plan:
        entries, end, spans = [], [], []
        for k, n in step:
            a = at[k]
            entries.append((k, seqs[k][a:a + n], list(range(n))))
            spans.append((k, a, n))
            at[k] = a + n
            if at[k] == len(seqs[k]):
                end.append(k)
        got = eng.step_tokens(entries, end)
        o = 0
        for k, a, n in spans:
            gots.append(got[o:o + n].cpu())
            refs.append(ref[k][a:a + n])
            o += n
        used.add(eng.bm.num_free_state_slots)
    assert all(at[k] == len(seqs[k]) for k in seqs)
    assert _err(torch.cat(gots), torch.cat(refs), dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4 and min(used) == 1
    with pytest.raises(RuntimeError):  # a fifth live sequence: no state slot
        eng.step_tokens([(k, [1, 2], []) for k in "vwxyz"])


def test_every_pass_of_a_loop_has_its_own_cache_and_state(gpu, tmp_path):
    """Looped layers share weights, not pages or state: with the loop the model differs from the same layers run
    once, and decoding after a prompt (which reads every pass's cache and state) matches the oracle's loop."""
    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32)
    assert len(model.runs) == 8 and len(model.cache_index) == 4 and len(model.state_fields()) == 4
    toks = _tokens(40, cfg["vocab"], 12)
    ref = O.forward(cfg, W, toks)
    once = O.forward({**cfg, "loop": None}, W, toks)
    assert float((ref - once).abs().max()) > 0.1
    got = [eng.step_tokens([("l", toks[:21], list(range(21)))])]
    for i in range(21, 40):
        got.append(eng.step_tokens([("l", [toks[i]], [0])], ["l"] if i == 39 else []))
    assert _err(torch.cat(got), ref) < TOL[torch.float32]


def test_long_decoding(gpu, tmp_path):
    """220 tokens decoded one by one after a short prompt (pages cross, the retention state runs long): fp32 stays at
    rounding distance from the oracle."""
    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, num_blocks=20, max_model_len=320)
    toks = _tokens(230, cfg["vocab"], 9)
    ref = O.forward(cfg, W, toks)
    got = [eng.step_tokens([("l", toks[:10], list(range(10)))])]
    for i in range(10, 230):
        got.append(eng.step_tokens([("l", [toks[i]], [0])], ["l"] if i == 229 else []))
    assert _err(torch.cat(got), ref) < TOL[torch.float32]


def _check_greedy(cfg, W, prompt, got, slack=0.04):
    """Every generated token is the oracle's best next token GIVEN the engine's own tokens so far, up to near-ties
    (the sampler reads bf16 logits: two logits closer than their rounding may swap); most are the exact argmax."""
    lg = O.forward(cfg, W, list(prompt) + list(got[:-1]))[len(prompt) - 1:]
    exact = 0
    for t, tok in enumerate(got):
        assert 0 <= tok < cfg["vocab"]
        assert float(lg[t].max() - lg[t, tok]) < slack, f"token {t}: {tok} is {float(lg[t].max() - lg[t, tok])} below the best"
        exact += int(lg[t].argmax()) == tok
    assert exact >= 0.8 * len(got)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_scheduler(gpu, tmp_path, graphs):
    """engine.generate (admission, paged prefill, state slots from the block manager, batched decode steps, the fused
    sampler at temperature 0; with hipGraph replay of the decode step when ``graphs``: its warm-up run must not advance
    the sequences' states) against the oracle's greedy continuation, twice on one engine so that slots and pages come
    back dirty."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, use_graphs=graphs, num_blocks=40)
    for seeds in ((21, 22), (23, 24)):
        prompts = [_tokens(23, 250, seeds[0]), _tokens(5, 250, seeds[1])]
        n_new = 40
        out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True))
        for p, o in zip(prompts, out):
            assert len(o[0]) == n_new
            _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


def test_generation_chunked_prefill_and_forks(gpu, tmp_path):
    """Chunked prefill (prompt portions beside running decodes) and n > 1 (forked sequences: shared prompt pages, the
    prompt's recurrent state copied to every child) give the greedy continuation too."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32, num_blocks=48, chunked_prefill=8, max_batch=8)
    prompts = [_tokens(37, 250, 31), _tokens(12, 250, 32)]
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True), n=2)
    for p, o in zip(prompts, out):
        assert len(o) == 2 and o[0] == o[1]  # greedy forks of one prompt agree
        _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 8


def test_server_worker_factory_builds_the_design(gpu, tmp_path):
    """The server's worker factory on a model folder of the design: prefix caching is switched off for it (a cached
    head brings no recurrent state), the state pool is there, generation works."""
    from llm_weighted_consensus_amd.engine.group import build_engine
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W = _make("mixed", 2)
    eng = build_engine({"model_dir": _save(tmp_path / "m", cfg, W), "dtype": "float32", "max_batch": 4, "max_model_len": 128,
                        "kv_fraction": 0.001}, 0)
    assert eng.state is not None and not eng.prefix_caching and eng.bm.num_state_slots == 4
    prompt = _tokens(20, cfg["vocab"], 8)
    out = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    _check_greedy(cfg, W, prompt, out[0][0])


def test_trace_replay_command_line(gpu, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, ``done <step>`` lines and <step>.f32 files out; two sequences
    interleaved (portions beside single tokens, one sitting a step out), pages and slots given back at ``end``."""
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, W = _make("mixed", 4)
    mdir, out = _save(tmp_path / "model", cfg, W), tmp_path / "out"
    a, b = _tokens(40, cfg["vocab"], 1), _tokens(21, cfg["vocab"], 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:20], "want": []}, {"id": "a", "tokens": a[30:31], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[31:], "want": [8, 2]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", mdir, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    ra, rb = O.forward(cfg, W, a), O.forward(cfg, W, b)
    want = {0: ra[[0, 29]], 2: rb[[20]], 3: ra[[39, 33]], 1: ra[[30]]}
    for step, ref in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4")).view(-1, cfg["vocab"])
        assert _err(got, ref) < TOL[torch.float32]
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32", "3.f32"]


def test_loader_refuses_wrong_shapes(gpu, tmp_path):
    from llm_weighted_consensus_amd.models.registry import load_model

    cfg, W = _make("odd", 0)
    bad = dict(W)
    bad["l0.mix.sink"] = torch.zeros(5, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        load_model(_save(tmp_path / "bad", cfg, bad))
    del bad["l1.mlp.gate"]
    bad["l0.mix.sink"] = W["l0.mix.sink"]
    with pytest.raises(KeyError):
        load_model(_save(tmp_path / "bad2", cfg, bad))
