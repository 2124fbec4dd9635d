"""Rerozen on the GPU against the plain fp64 oracle (tests/rerozen_oracle.py): each mechanism alone, then the model
through the engine — whole prompts, token-by-token decoding, portions, unequal batches, pages and state slots used
again, the first tokens of a sequence, keys just inside and just outside a chunk, far keys at page borders, long
decoding and greedy generation through the scheduler.  Small configurations with random weights, sizes chosen so that
nothing the design allows to differ happens to be equal or 1."""
import json
import math

import pytest
import torch

import rerozen_oracle as O

pytestmark = pytest.mark.gpu

F64 = torch.float64


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


def _paged(n_tokens, bs, nk, nv, dtype, perm_seed=0):
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache

    nb = -(-n_tokens // bs) + 3
    cache = PagedLayerCache([(nk, nv)], nb, bs, "cuda", dtype)
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(perm_seed))[: -(-n_tokens // bs)]
    slots = torch.tensor([int(perm[t // bs]) * bs + t % bs for t in range(n_tokens)], dtype=torch.int32)
    return cache, perm.to(torch.int32), slots


def _attend(res32, q, cache, pos, table, H, G, chunk, sink, out, a, c, gpu):
    """Rows [a, a + c) of one sequence: a single row as a decode row, more as a prompt portion."""
    z = torch.zeros(H, device=gpu)
    kw = dict(cores=True, sink=torch.zeros(H, device=gpu) if sink else None, chunk=chunk)
    if c > 1:
        kw.update(cu_q=torch.tensor([0, c], dtype=torch.int32, device=gpu),
                  k_lens=torch.tensor([a + c], dtype=torch.int32, device=gpu), max_q=c)
    res32.window_attn(q, cache.k[0], cache.v[0], pos, table, z, z, 1 << 30, out, H, G, **kw)


# ------------------------------------------------------------------ mechanisms, one by one
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 4e-2)])
@pytest.mark.parametrize("H,G,D,Dv,rd,chunk,two", [(4, 2, 12, 10, 8, 7, True), (2, 1, 16, 24, 16, 20, False), (3, 3, 10, 7, 0, 1, False),
                                                   (4, 2, 64, 64, 32, 24, True), (2, 2, 32, 32, 32, 16, False),
                                                   (8, 2, 128, 128, 64, 33, True), (4, 1, 128, 64, 128, 100, True)])
def test_rotary_cache_write_and_chunked_attention(gpu, dtype, tol, H, G, D, Dv, rd, chunk, two):
    """Per-head q / k norms (or none), rotation of the first ``rd`` entries with scaled frequencies at positions from 900
    on, values rotated on their way into the cache and the output turned back, chunked softmax with and without the
    sink, the per-head gate: a sequence written and attended in portions and single rows over shuffled pages (general
    kernel; matrix-core kernels for the sizes they take), against the oracle."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(H * 100 + D)
    n, bs, scale, eps, p0 = 75, 16, 0.31, 1e-5, 0
    nq, nk, nv = H * D, G * D, G * Dv
    dt_in = dtype if not two else torch.float32          # behind a convolution the rows are fp32
    src = (torch.randn(n, nq + nk + nv, generator=g) * 1.5).to(dt_in)
    gate = torch.randn(n, H, generator=g).to(dtype)
    wq, wk = (None, None) if two else (1 + 0.2 * torch.randn(D, generator=g), 1 + 0.2 * torch.randn(D, generator=g))
    scaling = dict(factor=4.0, original=64, fast=8.0, slow=2.0) if two else None
    pos = torch.arange(p0, p0 + n)
    q, k, v = src[:, :nq].double().view(n, H, D), src[:, nq:nq + nk].double().view(n, G, D), src[:, nq + nk:].double().view(n, G, Dv)
    if not two:
        q, k = O.rms_norm(q, wq.double(), eps), O.rms_norm(k, wk.double(), eps)
    f = mult = None
    if rd:
        f, mult = O.rope_freqs(rd, 5000.0, scaling)
        q, k = O.rotate(q, pos, f, mult), O.rotate(k, pos, f, mult)
    fv = O.rope_freqs(Dv, 5000.0)[0] if two else None
    if two:
        v = O.rotate(v, pos, fv)
    ref = O.chunked_softmax_attention(q, k, v, scale, chunk, sink=two)
    if two:
        ref = O.rotate(ref, pos, fv, sign=-1.0)
    ref = (ref * torch.sigmoid(gate.double())[:, :, None] * 0.6).reshape(n, H * Dv)

    cache, table, slots = _paged(p0 + n, bs, nk, nv, dtype, 3)
    fg = res32.rope_frequencies(rd, 5000.0, scaling, gpu) if rd else (None, 1.0)
    fvg = res32.rope_frequencies(Dv, 5000.0, None, gpu)[0] if two else None
    if rd:
        assert (fg[0].cpu().double() - f).abs().max() < 1e-7 and abs(fg[1] - mult) < 1e-12
    table_g, posg = table.to(gpu)[None], pos.to(torch.int32).to(gpu)
    outs, a = [], 0
    for c in [17, 2, 1, 1, 9, 15, 1, 29]:
        rows = slice(a, a + c)
        qo = res32.rot_kv_write(src[rows].to(gpu), posg[rows], slots[p0:][rows].to(gpu), cache.k[0], cache.v[0], H, G, scale,
                                rot_dims=rd, freq=fg[0], mult=fg[1], vfreq=fvg, wq=None if two else wq.to(gpu),
                                wk=None if two else wk.to(gpu), eps=eps)
        assert (qo.cpu().double().view(c, H, D) - q[rows] * scale).abs().max() < (3e-4 if dtype == torch.float32 else 0.2)
        o = torch.empty(c, H * Dv, dtype=dtype, device=gpu)
        _attend(res32, qo, cache, posg[rows], table_g, H, G, chunk, two, o, a + p0, c, gpu)
        out = torch.empty(c, H * Dv + 3, dtype=dtype, device=gpu)[:, 3:]   # a column slice, as in the model
        res32.head_gate_unrotate(o, out, posg[rows], H, gate=gate[rows].to(gpu), vfreq=fvg, scale=0.6)
        outs.append(out.cpu())
        a += c
    assert a == n
    assert (torch.cat(outs).double() - ref).abs().max() < tol * 8
    kc, vc = cache.rows(0, slots[p0:].long().to(gpu))
    assert (kc.cpu().double() - k.reshape(n, nk)).abs().max() < tol * 4
    assert (vc.cpu().double() - v.reshape(n, nv)).abs().max() < tol * 6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_at_large_positions(gpu, dtype):
    """Angles are fp32 products position * frequency: keys written at positions 900 .. 1000 match the oracle's rotation."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(5)
    H, G, D, Dv, n, p0 = 2, 1, 24, 8, 101, 900
    src = torch.randn(n, H * D + G * D + G * Dv, generator=g).to(dtype)
    pos = torch.arange(p0, p0 + n)
    f, mult = O.rope_freqs(16, 10000.0, dict(factor=3.0, original=512, fast=16.0, slow=1.0))
    cache, table, slots = _paged(p0 + n, 16, G * D, G * Dv, dtype, 1)
    fg = res32.rope_frequencies(16, 10000.0, dict(factor=3.0, original=512, fast=16.0, slow=1.0), gpu)
    qo = res32.rot_kv_write(src.to(gpu), pos.to(torch.int32).to(gpu), slots[p0:].to(gpu), cache.k[0], cache.v[0], H, G, 1.0,
                            rot_dims=16, freq=fg[0], mult=fg[1])
    ref_q = O.rotate(src[:, :H * D].double().view(n, H, D), pos, f, mult)
    ref_k = O.rotate(src[:, H * D:H * D + G * D].double().view(n, G, D), pos, f, mult)
    assert (qo.cpu().double().view(n, H, D) - ref_q).abs().max() < 5e-4   # fp32 angles near 1000 radians
    kc, _ = cache.rows(0, slots[p0:].long().to(gpu))
    assert (kc.cpu().double().view(n, G, D) - ref_k).abs().max() < (5e-4 if dtype == torch.float32 else 3e-2)
    assert (ref_q[:, :, 16:] - src[:, :H * D].double().view(n, H, D)[:, :, 16:]).abs().max() == 0   # the rest passes


@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk", [48, 100])
def test_chunk_edges_and_page_borders_stand_out(gpu, decode, dtype, chunk):
    """Among 300 keys over shuffled pages one query matches ONE key strongly.  Inside the row's chunk (its first key, both
    sides of page borders, the row itself) the output is that key's value; one key OUTSIDE the chunk (the last of the
    chunk before) is not seen however well it matches: the output is then the flat mean of the chunk's values (head 1
    shows that flat mean throughout).  With the sink of score 0 a flat head's weights sum to n / (n + 1)."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(11)
    n, bs, H, G, D = 300, 16, 2, 1, 32
    k = torch.randn(n, D, generator=g).to(torch.bfloat16)
    kn = k.double() / k.double().norm(dim=-1, keepdim=True)
    cache, table, slots = _paged(n, bs, D, D, dtype, 5)
    cache.set_rows(0, slots.long().to(gpu), kn.to(dtype).to(gpu), k.to(dtype).to(gpu))
    z = torch.zeros(H, device=gpu)
    for i in (n - 1, 2 * chunk, 2 * chunk - 1, chunk + 17):
        lo = i - i % chunk
        inside = sorted({lo, min(lo + 1, i), i, *[j for j in (lo + 15, lo + 16, lo + 17, i - 1) if lo <= j <= i]})
        for sink in (False, True):
            for j in inside + [lo - 1]:
                q = torch.zeros(1, H * D)
                q[0, :D] = kn[j].float() * 40  # head 0 looks for key j; head 1 sees a flat softmax
                out = torch.empty(1, H * D, dtype=dtype, device=gpu)
                pos = torch.tensor([i], dtype=torch.int32, device=gpu)
                kw = {} if decode else dict(cu_q=torch.tensor([0, 1], dtype=torch.int32, device=gpu),
                                            k_lens=torch.tensor([i + 1], dtype=torch.int32, device=gpu), max_q=1)
                res32.window_attn(q.to(gpu), cache.k[0], cache.v[0], pos, table.to(gpu)[None], z, z, 1 << 30, out, H, G,
                                  cores=True, sink=z if sink else None, chunk=chunk, **kw)
                seen = k[lo:i + 1].double()
                flat = seen.sum(0) / (seen.shape[0] + (1 if sink else 0))
                assert (out[0, D:].cpu().double() - flat).abs().max() < 0.05, (i, j, sink)
                if j >= lo:
                    assert (out[0, :D].cpu().double() - k[j].double()).abs().max() < 0.06, (i, j, sink)
                else:   # its score would be 40 against about 40 * 0.2 for the others: seen, it would take everything
                    assert (out[0, :D].cpu().double() - k[j].double()).abs().max() > 0.5, (i, j, sink)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("chunk,D,Dv", [(40, 64, 64), (64, 20, 12), (13, 128, 128)])
def test_chunked_portions_of_several_sequences(gpu, dtype, tol, chunk, D, Dv):
    """Prompt portions of two sequences in one call, cut inside chunks and at their edges, rows of one tile belonging to
    different chunks (the matrix-core portion kernel for the sizes it takes), with the sink."""
    from llm_weighted_consensus_amd.models.cache import PagedLayerCache
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(chunk)
    H, G, bs, lens = 4, 2, 16, [150, 90]
    cache = PagedLayerCache([(G * D, G * Dv)], 20, bs, "cuda", dtype)
    perm = torch.randperm(20, generator=g)
    tables = torch.stack([perm[:10], perm[10:]]).to(torch.int32)
    seqs = []
    for s, n in enumerate(lens):
        q = torch.randn(n, H, D, generator=g).to(torch.bfloat16).double()
        k = torch.randn(n, G, D, generator=g).to(torch.bfloat16).double()
        v = torch.randn(n, G, Dv, generator=g).to(torch.bfloat16).double()
        slots = torch.tensor([int(tables[s, t // bs]) * bs + t % bs for t in range(n)])
        cache.set_rows(0, slots.to(gpu), k.reshape(n, -1).to(gpu), v.reshape(n, -1).to(gpu))
        seqs.append((q, O.chunked_softmax_attention(q, k, v, 0.2, chunk, sink=True).reshape(n, H * Dv)))
    z = torch.zeros(H, device=gpu)
    for cuts in ([(0, 70), (0, 90)], [(70, 150), (3, 5)], [(chunk - 1, chunk + 2), (chunk, min(2 * chunk, 90))], [(37, 38), (1, 66)]):
        q = torch.cat([seqs[s][0][a:b].reshape(b - a, H * D) * 0.2 for s, (a, b) in enumerate(cuts)]).float().to(gpu)
        pos = torch.cat([torch.arange(a, b) for a, b in cuts]).to(torch.int32).to(gpu)
        ql = [b - a for a, b in cuts]
        out = torch.empty(sum(ql), H * Dv, dtype=dtype, device=gpu)
        res32.window_attn(q, cache.k[0], cache.v[0], pos, tables.to(gpu), z, z, 1 << 30, out, H, G,
                          cu_q=torch.tensor([0, ql[0], sum(ql)], dtype=torch.int32, device=gpu),
                          k_lens=torch.tensor([b for _, b in cuts], dtype=torch.int32, device=gpu), max_q=max(ql), cores=True,
                          sink=z, chunk=chunk)
        ref = torch.cat([seqs[s][1][a:b] for s, (a, b) in enumerate(cuts)])
        assert (out.cpu().double() - ref).abs().max() < tol * 4, cuts


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
def test_plain_convolution_with_history(gpu, dtype, tol):
    """conv(x) without activation in portions down to one row, in a slot that held other data."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(2)
    for taps, C in ((3, 37), (2, 40), (1, 12), (5, 264)):
        n = 30
        x = torch.randn(n, C, generator=g).to(dtype)
        w = torch.randn(C, taps, generator=g)
        ref = O.causal_conv(x.double(), w.double())
        hist = torch.randn(3, taps - 1, C, generator=g).to(gpu) * 50
        wg = w.to(gpu).t().contiguous().t()
        outs, a = [], 0
        for c in (1, 2, 1, 9, 17):
            out = torch.empty(c, C, dtype=torch.float32, device=gpu)
            res32.conv_hist(x[a:a + c].to(gpu), wg, hist, _items([c], [1], [a], gpu), out, mode=2)
            outs.append(out.cpu())
            a += c
        assert (torch.cat(outs).double() - ref).abs().max() < tol * 8, (taps, C)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,delta", [(4, 2, 12, 20, True), (3, 3, 8, 6, False), (2, 1, 70, 66, True), (2, 2, 32, 32, False),
                                            (1, 1, 130, 16, False), (4, 4, 64, 128, True)])
def test_channel_decay_recurrences(gpu, dtype, H, G, D, Dv, delta):
    """Both recurrences with a decay per head and key channel: two sequences in portions down to one row, interleaved in
    one step, in slots that held other data; the state a portion leaves is the oracle's."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(H + D + Dv)
    lens = {"a": 37, "b": 11}
    fp = dtype == torch.float32
    data, ref, Sref = {}, {}, {}
    A_log = torch.rand(H, generator=g) * 2 - 2
    zb = torch.randn(H * D, generator=g) + (0.0 if delta else 2.0)
    tau = 6.5
    for s, n in lens.items():
        src = torch.randn(n, 2 * G * D + H * Dv, generator=g).to(torch.float32 if delta else dtype)
        z = torch.randn(n, H * D, generator=g)
        b = torch.randn(n, H, generator=g).to(dtype)
        data[s] = (src, z, b)
        q, k = src[:, :G * D].double().view(n, G, D), src[:, G * D:2 * G * D].double().view(n, G, D)
        v = src[:, 2 * G * D:].double().view(n, H, Dv)
        if delta:
            q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6)
            k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            dec = torch.exp(-torch.exp(A_log.double())[None, :, None] * torch.nn.functional.softplus((z.double() + zb.double()).view(n, H, D)))
        else:
            dec = (torch.sigmoid(z.double() + zb.double()) ** (1 / tau)).view(n, H, D)
        q = (q * D ** -0.5).repeat_interleave(H // G, 1)
        ref[s], Sref[s] = O.recurrence(q, k.repeat_interleave(H // G, 1), v, dec, torch.sigmoid(b.double()) if delta else None)
    state = (torch.randn(4, H, D, Dv, generator=g) * 30).to(gpu)
    plan = [[("a", 1)], [("a", 2), ("b", 1)], [("b", 2), ("a", 1)], [("a", 7)], [("b", 8), ("a", 26)]]
    at, got, slot = {"a": 0, "b": 0}, {"a": [], "b": []}, {"a": 2, "b": 0}
    for step in plan:
        cat = lambda i: torch.cat([data[s][i][at[s]:at[s] + n] for s, n in step]).to(gpu)  # noqa: E731
        items = _items([n for _, n in step], [slot[s] for s, _ in step], [at[s] for s, _ in step], gpu)
        o = res32.channel_decay_rule(cat(0), cat(1), state, items, H, G, zb=zb.to(gpu), A_log=A_log.to(gpu) if delta else None,
                                     tau=tau, beta=cat(2) if delta else None, unit=delta, delta=delta)
        a = 0
        for s, n in step:
            got[s].append(o[a:a + n].cpu())
            a, at[s] = a + n, at[s] + n
    assert at == lens
    tol = 2e-4 if fp or delta else 3e-2
    for s in lens:
        scale = ref[s].abs().max().clamp_min(1.0)
        assert (torch.cat(got[s]).double().view(-1, H, Dv) - ref[s]).abs().max() / scale < tol, s
        assert (state[slot[s]].cpu().double() - Sref[s]).abs().max() / Sref[s].abs().max().clamp_min(1.0) < tol, s


@pytest.mark.parametrize("delta", [False, True])
def test_channel_decay_many_sequences_at_once(gpu, delta):
    """64 sequences side by side, two steps each (a grid large enough for the quarter-column split at D = 64): a portion
    of three rows, then single rows, against the oracle."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(3)
    B, H, G, D, Dv, n = 64, 8, 4, 64, 64, 5
    src = torch.randn(B, n, 2 * G * D + H * Dv, generator=g)
    z = torch.randn(B, n, H * D, generator=g) + 2.0
    b = torch.randn(B, n, H, generator=g)
    A_log = torch.rand(H, generator=g) - 2
    state = (torch.randn(B + 1, H, D, Dv, generator=g) * 9).to(gpu)
    slots = torch.randperm(B, generator=g).tolist()
    got = torch.empty(B, n, H * Dv)
    for a, c in ((0, 3), (3, 1), (4, 1)):
        rows = lambda x: x[:, a:a + c].reshape(B * c, -1).contiguous().to(gpu)  # noqa: E731
        o = res32.channel_decay_rule(rows(src), rows(z), state, _items([c] * B, slots, [a] * B, gpu), H, G,
                                     A_log=A_log.to(gpu) if delta else None, tau=3.0, beta=rows(b) if delta else None,
                                     unit=delta, delta=delta)
        got[:, a:a + c] = o.cpu().view(B, c, H * Dv)
    for s in (0, 17, 63):
        q, k = src[s, :, :G * D].double().view(n, G, D), src[s, :, G * D:2 * G * D].double().view(n, G, D)
        v = src[s, :, 2 * G * D:].double().view(n, H, Dv)
        if delta:
            q, k = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6), k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            dec = torch.exp(-torch.exp(A_log.double())[None, :, None] * torch.nn.functional.softplus(z[s].double().view(n, H, D)))
        else:
            dec = (torch.sigmoid(z[s].double()) ** (1 / 3.0)).view(n, H, D)
        ref, S = O.recurrence((q * D ** -0.5).repeat_interleave(H // G, 1), k.repeat_interleave(H // G, 1), v, dec,
                              torch.sigmoid(b[s].double()) if delta else None)
        assert (got[s].double().view(n, H, Dv) - ref).abs().max() / ref.abs().max().clamp_min(1.0) < 2e-4, s
        assert (state[slots[s]].cpu().double() - S).abs().max() / S.abs().max().clamp_min(1.0) < 2e-4, s


def test_far_token_survives_a_slow_decay(gpu):
    """A value written 400 tokens back under decays near one is read out with its exact weight: the product of the
    decays of its key channel since then (nothing else is written on that channel)."""
    from llm_weighted_consensus_amd.ops import res32

    n, H, D, Dv = 401, 1, 8, 4
    src = torch.zeros(n, 2 * D + Dv)
    src[0, D + 3], src[0, 2 * D:] = 1.0, torch.tensor([1.0, -2.0, 3.0, 0.5])       # k = e_3, v at the first token
    src[1:, D + 5] = 1.0                                                            # later tokens write channel 5
    src[1:, 2 * D:] = 7.0
    src[-1, 3] = math.sqrt(D)                                                       # the last query reads channel 3
    z = torch.full((n, D), 6.0)
    state = torch.randn(2, H, D, Dv).to(gpu)
    out = []
    for a, c in ((0, 1), (1, 250), (251, 149), (400, 1)):
        out.append(res32.channel_decay_rule(src[a:a + c].to(gpu), z[a:a + c].to(gpu), state, _items([c], [1], [a], gpu), H, H, tau=2.0).cpu())
    want = torch.sigmoid(torch.tensor(6.0, dtype=F64)) ** (400 / 2.0) * torch.tensor([1.0, -2.0, 3.0, 0.5], dtype=F64)
    assert (out[-1][0].double() - want).abs().max() < 1e-4   # 400 fp32 products in a row


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels(gpu, dtype):
    """erf gelu, residual add + norm, scaled embedding rows."""
    from llm_weighted_consensus_amd.ops import res32

    g = torch.Generator().manual_seed(0)
    for d in (37, 40, 1032):
        z = (torch.randn(9, d, generator=g) * 3).to(dtype)
        tol = 1e-6 if dtype == torch.float32 else 2e-2
        assert (res32.gelu(z.to(gpu)).cpu().double() - O.gelu_erf(z.double())).abs().max() < tol * 4
        x, w = torch.randn(9, d, generator=g) * 4, 1 + 0.1 * torch.randn(d, generator=g)
        xg = x.to(gpu)
        for out_dt in (torch.float32, dtype):
            xg.copy_(x)
            n = res32.add_rmsnorm(xg, z.to(gpu), w.to(gpu), 1e-5, out_dt)
            s = x.double() + z.double()
            assert (xg.cpu().double() - s).abs().max() < 1e-6
            assert (n.cpu().double() - O.rms_norm(s, w.double(), 1e-5)).abs().max() < (1e-5 if out_dt == torch.float32 else 3e-2)
        n = res32.add_rmsnorm(xg, None, w.to(gpu), 1e-5, torch.float32)
        assert (n.cpu().double() - O.rms_norm(xg.cpu().double(), w.double(), 1e-5)).abs().max() < 1e-5
    table = torch.randn(20, 37, generator=g).to(dtype)
    toks = torch.tensor([3, 19, 0], dtype=torch.int32)
    assert (res32.embed_rows(table.to(gpu), toks.to(gpu), scale=5.5).cpu().double() - table[toks.long()].double() * 5.5).abs().max() < 1e-5


# ------------------------------------------------------------------ the model through the engine
def _p2(left, right, **kw):
    return dict(type="parallel_2", left=left, right=right, **kw)


def _p1(left, right, **kw):
    return dict(type="parallel", left=left, right=right, **kw)


YARN = dict(factor=4.0, original=64, fast=8.0, slow=2.0)
CONFIGS = {
    # both layer kinds at different sizes; a layer without feed-forward; GQA on both sides; conv taps != canon taps
    "mixed": dict(width=40, vocab=250, taps=3, layers=[
        _p2(O.attention_left(4, 2, 12, 10, 7, 8, conv=2, scaling=YARN), dict(heads=4, kv_heads=2, dim=12, vdim=20, conv=2), ff=24),
        _p1(O.attention_left(2, 1, 16, 24, 20, 16, base=5000.0), dict(heads=3, dim=8, vdim=6, tau=4.0), ff=None, left_scale=1.2,
            right_scale=0.4, a_rank=3),
        _p1(O.attention_left(3, 3, 10, 10, 33, 4, scaling=dict(factor=2.0, original=32, fast=4.0, slow=1.0)),
            dict(heads=2, dim=20, vdim=12, tau=9.5), ff=16),
        _p2(O.attention_left(2, 2, 8, 8, 16, 8, conv=4), dict(heads=2, kv_heads=2, dim=8, vdim=8, conv=4), ff=None, g_rank=2)]),
    # odd sizes; one tap everywhere (no histories); no rotation in one layer; one head; a chunk of one token and one
    # longer than any sequence
    "odd": dict(width=34, vocab=131, taps=1, layers=[
        _p1(O.attention_left(1, 1, 10, 7, 1, 0), dict(heads=1, dim=5, vdim=9, tau=1.0), ff=9),
        _p2(O.attention_left(3, 1, 6, 6, 1000, 2, conv=1), dict(heads=3, kv_heads=1, dim=70, vdim=66, conv=1), ff=None),
        _p2(O.attention_left(2, 2, 14, 4, 5, 14, conv=3, base=300.0), dict(heads=2, kv_heads=2, dim=7, vdim=3, conv=2), ff=11)]),
    # sizes the matrix-core attention kernels take
    "cores": dict(width=64, vocab=320, taps=4, layers=[
        _p2(O.attention_left(4, 2, 64, 64, 48, 32, conv=3, scaling=YARN), dict(heads=2, kv_heads=1, dim=64, vdim=64, conv=3), ff=64),
        _p1(O.attention_left(2, 2, 32, 32, 16, 32), dict(heads=4, dim=32, vdim=32, tau=8.0), ff=32),
        _p2(O.attention_left(8, 2, 128, 128, 100, 64, conv=2), dict(heads=4, kv_heads=4, dim=32, vdim=64, conv=4), ff=None),
        _p1(O.attention_left(4, 1, 128, 64, 40, 128), dict(heads=2, dim=64, vdim=32, tau=16.0), ff=None)]),
}


def _build(tmp_path, name, dtype, seed=0, **engine_kw):
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.engine.engine import LLMEngine
    from llm_weighted_consensus_amd.engine.tokenizer import load_tokenizer
    from llm_weighted_consensus_amd.models.registry import load_model

    c = CONFIGS[name]
    cfg, ranks = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"])
    W = O.make_weights(cfg, ranks, seed)
    d = tmp_path / f"{name}-{seed}"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    model = load_model(str(d), dtype=dtype)
    kw = dict(block_size=16, num_blocks=24, max_batch=4, max_model_len=256, use_graphs=False, prefix_sharing=False,
              tune_gc=False)
    kw.update(engine_kw)
    return cfg, W, model, LLMEngine(model, load_tokenizer({}, cfg["vocab"]), **kw)


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _err(got, ref, dtype=torch.float32):
    """fp32: the largest difference.  bf16: the row-wise relative RMS difference that 90 % of the rows stay under,
    times 4, and no row may be off by more than its own size."""
    d, ref = got.cpu().double() - ref, ref.double()
    if dtype == torch.float32:
        return float(d.abs().max())
    rel = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert float(rel.max()) < 1.0
    return 4 * float(rel.flatten().quantile(0.9))


TOL = {torch.float32: 3e-4, torch.bfloat16: 0.5}


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("mixed", torch.bfloat16), ("odd", torch.float32),
                                        ("odd", torch.bfloat16), ("cores", torch.float32), ("cores", torch.bfloat16)])
def test_whole_prompt_and_every_layer(gpu, tmp_path, name, dtype):
    """A whole prompt in one step: the stream after every layer and the logits against the oracle."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(150, cfg["vocab"], 1)
    layers = []
    ref = O.forward(cfg, W, toks, layers)
    seen = []
    model.on_layer = lambda li, x: seen.append(x.detach().cpu().double())
    got = eng.step_tokens([("w", toks, list(range(len(toks))))], ["w"])
    model.on_layer = None
    assert len(seen) == len(layers)
    for li, (a, b) in enumerate(zip(seen, layers)):
        assert _err(a, b, dtype) < TOL[dtype] * (4 if dtype == torch.float32 else 0.2), li
    assert _err(got, ref, dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("mixed", torch.bfloat16), ("cores", torch.bfloat16), ("odd", torch.float32)])
def test_token_by_token_and_portions(gpu, tmp_path, name, dtype):
    """The same sequence decoded one token at a time from its first token, and in portions of several sizes down to two
    tokens (cut inside chunks, pages and convolution histories), equals the whole prompt's oracle."""
    cfg, W, model, eng = _build(tmp_path, name, dtype)
    toks = _tokens(77, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    rows = [eng.step_tokens([("d", [t], [0])], ["d"] if i + 1 == len(toks) else []) for i, t in enumerate(toks)]
    assert _err(torch.cat(rows), ref, dtype) < TOL[dtype]
    for sizes in ([2, 2, 13, 3, 16, 2, 30, 9], [17, 16, 15, 2, 27], [1, 2, 5, 69]):
        assert sum(sizes) == len(toks)
        rows, a = [], 0
        for n in sizes:
            rows.append(eng.step_tokens([("p", toks[a:a + n], list(range(n)))], ["p"] if a + n == len(toks) else []))
            a += n
        assert _err(torch.cat(rows), ref, dtype) < TOL[dtype]
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


@pytest.mark.parametrize("name,dtype", [("mixed", torch.float32), ("mixed", torch.bfloat16), ("cores", torch.bfloat16)])
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


def test_the_chunk_matters_at_its_edges(gpu, tmp_path):
    """The oracle with every chunk size changed by one differs from the right one exactly from the first position where
    the two masks differ; the engine follows the right one there, in a prompt and decoded one by one."""
    cfg, W, model, eng = _build(tmp_path, "mixed", torch.float32)
    toks = _tokens(60, cfg["vocab"], 6)
    ref = O.forward(cfg, W, toks)
    off = json.loads(json.dumps(cfg))
    for L in off["layers"]:
        L["mixer"]["left"]["mask"]["size"] += 1
    ref1 = O.forward(off, W, toks)
    first = min(L["mixer"]["left"]["mask"]["size"] for L in cfg["layers"])   # position `first` opens the second chunk
    assert float((ref[:first] - ref1[:first]).abs().max()) < 1e-9 and float((ref[first] - ref1[first]).abs().max()) > 1e-3
    got = eng.step_tokens([("t", toks[:30], list(range(30)))])
    assert _err(got, ref[:30]) < TOL[torch.float32]
    for i in range(30, 60):
        got = eng.step_tokens([("t", [toks[i]], [0])], ["t"] if i == 59 else [])
        assert _err(got, ref[[i]]) < TOL[torch.float32]


def test_long_decoding_against_the_recurrence(gpu, tmp_path):
    """220 tokens decoded one by one after a short prompt (pages cross, many chunks pass, the states run long): fp32
    stays at rounding distance from the oracle."""
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
        out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True))
        for p, o in zip(prompts, out):
            assert len(o[0]) == 40
            _check_greedy(cfg, W, p, o[0])
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


def test_generation_chunked_prefill_and_forks(gpu, tmp_path):
    """Chunked prefill (prompt portions beside running decodes) and n > 1 (forked sequences: shared prompt pages, the
    prompt's recurrent state copied to every child) give the greedy continuation too."""
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    cfg, W, model, eng = _build(tmp_path, "cores", torch.bfloat16, num_blocks=48, chunked_prefill=8, max_batch=8)
    prompts = [_tokens(37, cfg["vocab"], 31), _tokens(12, cfg["vocab"], 32)]
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True), n=2)
    for p, o in zip(prompts, out):
        assert len(o) == 2 and o[0] == o[1]  # greedy forks of one prompt agree
        _check_greedy(cfg, W, p, o[0], slack=0.25)
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 8


def test_server_worker_factory_and_seeded_sampling(gpu, tmp_path):
    """The server's worker factory on a model folder of the design: prefix caching is off for it (a cached head brings
    no recurrent state), the state pool is there.  Seeded top-k sampling through the engine's sampler: the same seed
    gives the same tokens, and every drawn token is among the oracle's k best next tokens given the engine's own
    tokens so far (up to near-ties at the k-th place)."""
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.engine.group import build_engine
    from llm_weighted_consensus_amd.engine.sampling import SamplingParams

    c = CONFIGS["mixed"]
    cfg, ranks = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"])
    W = O.make_weights(cfg, ranks, 5)
    d = tmp_path / "served"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    eng = build_engine({"model_dir": str(d), "dtype": "float32", "max_batch": 4, "max_model_len": 128, "kv_fraction": 0.001}, 0)
    assert eng.state is not None and not eng.prefix_caching and eng.bm.num_state_slots == 4
    prompt = _tokens(20, cfg["vocab"], 8)
    out = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    _check_greedy(cfg, W, prompt, out[0][0])
    sp = SamplingParams(temperature=1.5, top_k=5, max_tokens=24, ignore_eos=True, seed=7)
    one, two = eng.generate([prompt], sp)[0][0], eng.generate([prompt], sp)[0][0]
    assert one == two and len(one) == 24
    lg = O.forward(cfg, W, prompt + one[:-1])[len(prompt) - 1:]
    for t, tok in enumerate(one):
        assert float(lg[t].topk(5).values[-1] - lg[t, tok]) < 0.04, t
    assert any(int(lg[t].argmax()) != tok for t, tok in enumerate(one))  # some draws are not the best token
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == 4


def test_trace_replay_command_line(gpu, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, ``done <step>`` lines and <step>.f32 files out; two sequences
    interleaved (portions beside single tokens, one sitting a step out), pages and slots given back at ``end``."""
    import os
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file

    c = CONFIGS["mixed"]
    cfg, ranks = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"])
    W = O.make_weights(cfg, ranks, 4)
    mdir, out = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(mdir / "model.safetensors"))
    a, b = _tokens(40, cfg["vocab"], 1), _tokens(21, cfg["vocab"], 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:20], "want": []}, {"id": "a", "tokens": a[30:31], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[31:], "want": [8, 2]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(mdir), "--dtype", "float32",
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
    from safetensors.torch import save_file

    from llm_weighted_consensus_amd.models.registry import load_model

    c = CONFIGS["odd"]
    cfg, ranks = O.make_config(c["width"], c["vocab"], c["layers"], taps=c["taps"])
    W = O.make_weights(cfg, ranks, 0)
    d = tmp_path / "bad"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    bad = dict(W)
    bad["l1.mix.right.A_log"] = torch.zeros(5, dtype=torch.bfloat16)
    save_file(bad, str(d / "model.safetensors"))
    with pytest.raises(ValueError):
        load_model(str(d))
    bad = dict(W)
    del bad["l0.mix.left.q.b"]
    save_file(bad, str(d / "model.safetensors"))
    with pytest.raises(KeyError):
        load_model(str(d))
