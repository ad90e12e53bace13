"""Each mechanism of the hybrid decoder alone: the framework's op (``ops`` dispatch; CPU here,
the HIP kernels in the ``gpu`` variants) against the matching function of the plain oracle.
Inputs are shaped so that a fault shows: one key far back (or at a page border, or one
position beyond what a query may see) given a score that dominates the softmax, a sink that
takes most of the weight, frequencies in each branch of the scaling rule, portions shorter
than the convolution, routing groups whose best expert is not the overall best."""
import math

import pytest
import torch

import natilix_oracle as orc
from minivllm_amd import ops

DEVICES = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]


def to(dev, *ts):
    return [t if t is None else t.to(dev) for t in ts]


@pytest.mark.parametrize("dev", DEVICES)
def test_norms_and_embedding(dev):
    torch.manual_seed(0)
    T, W = 7, 30
    x, w, y, wb = torch.randn(T, W), 0.3 * torch.randn(W), torch.randn(T, W), 0.3 * torch.randn(W)
    got = ops.offset_rms_norm(*to(dev, x, w), 1e-4, torch.float32).cpu()
    torch.testing.assert_close(got, orc.norm_around_zero(x.double(), w.double(), 1e-4).float())
    xs = x.clone().to(dev)
    h = ops.post_norm_residual(*to(dev, y, wb), xs, 1e-4, w.to(dev), torch.float32).cpu()
    want_x = x.double() + orc.norm_around_zero(y.double(), wb.double(), 1e-4)
    torch.testing.assert_close(xs.cpu(), want_x.float())
    torch.testing.assert_close(h, orc.norm_around_zero(want_x, w.double(), 1e-4).float())
    # bigram rows: first token of a sequence, a continued portion, arithmetic beyond 32 bits
    from minivllm_amd.layers.embedding_head import HashedBigramEmbedding
    e = HashedBigramEmbedding(101, 4, 2 ** 20 + 7, 2 ** 19 + 3)
    toks = [90000, 5, 70000, 70000]
    assert e.rows_for(toks, [-1] + toks[:-1]).tolist() == orc.bigram_rows(toks, None, e.mul_prev, e.mul_cur, 101)
    assert e.rows_for(toks[2:], toks[1:3]).tolist() == orc.bigram_rows(toks[2:], toks[1], e.mul_prev, e.mul_cur, 101)


def test_rotation_table_covers_every_branch_of_the_scaling_rule():
    from minivllm_amd.ops.torch_seqmix import pair_cos_sin_table
    sc = {"factor": 5.0, "low": 1.0, "high": 4.0, "original": 64}
    dims, base = 16, 500.0
    f = orc.rope_frequencies(dims, base, sc)
    plain = orc.rope_frequencies(dims, base, None)
    ratio = (f / plain).tolist()
    assert any(r == 1.0 for r in ratio) and any(abs(r - 0.2) < 1e-12 for r in ratio) \
        and any(0.2 + 1e-6 < r < 1 - 1e-6 for r in ratio), ratio
    table = pair_cos_sin_table(dims, 300, base, sc)
    pos = torch.arange(300)
    ang = (pos.float()[:, None] * f.float()[None]).double()
    torch.testing.assert_close(table, torch.cat([ang.cos(), ang.sin()], -1).float(), rtol=0, atol=1e-7)


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("rot,D", [(8, 8), (6, 10), (0, 4)])
def test_rotation_value_mix_and_store(dev, rot, D):
    from minivllm_amd.ops.torch_seqmix import pair_cos_sin_table
    torch.manual_seed(1)
    T, H, G, E, bs = 9, 4, 2, 6, 4
    sc = {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 8}
    proj = torch.randn(T, H * D + G * D + G * E)
    pos = torch.tensor([0, 1, 2, 3, 4, 37, 38, 200, 201], dtype=torch.int32)
    slots = torch.tensor([5, 6, 7, 0, 1, 12, 13, 2, 3], dtype=torch.int32)
    table = pair_cos_sin_table(rot, 256, 50.0, sc) if rot else None
    vf, lam = torch.randn(T, G, E), torch.tensor(0.6)
    p = proj.clone().to(dev)
    q, k, v = p.split([H * D, G * D, G * E], -1)
    kc, vc = torch.zeros(4, bs, G, D).to(dev), torch.zeros(4, bs, G, E).to(dev)
    ops.pair_rope_mix_store(q.view(T, H, D), k.view(T, G, D), v.view(T, G, E), pos.to(dev),
                            None if table is None else table.to(dev), rot, vf.to(dev), lam.to(dev), 2,
                            kc, vc, slots.to(dev))
    q0, k0, v0 = proj.double().split([H * D, G * D, G * E], -1)
    f = orc.rope_frequencies(rot, 50.0, sc) if rot else None
    wq = orc.rope_pairs(q0.view(T, H, D), pos, f, rot) if rot else q0.view(T, H, D)
    wk = orc.rope_pairs(k0.view(T, G, D), pos, f, rot) if rot else k0.view(T, G, D)
    wv = 0.4 * v0.view(T, G, E) + 0.6 * vf.double()
    torch.testing.assert_close(q.cpu().view(T, H, D), wq.float(), rtol=1e-5, atol=1e-5)
    sl = slots.long()
    torch.testing.assert_close(kc.cpu().view(-1, G, D)[sl], wk.float(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(vc.cpu().view(-1, G, E)[sl], wv.float(), rtol=1e-5, atol=1e-5)


def _cache_from(k, v, bs, perm_seed=0):
    """Scatter one sequence's K [L,G,D] / V [L,G,E] into a paged cache with shuffled blocks."""
    L = k.shape[0]
    nb = (L + bs - 1) // bs
    g = torch.Generator().manual_seed(perm_seed)
    table = torch.randperm(nb + 2, generator=g)[:nb].to(torch.int32)
    kc, vc = torch.zeros(nb + 2, bs, *k.shape[1:]), torch.zeros(nb + 2, bs, *v.shape[1:])
    for j in range(L):
        kc[table[j // bs], j % bs], vc[table[j // bs], j % bs] = k[j], v[j]
    return kc, vc, table[None]


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("far", [0, 1, 15, 16, 17, 255, 256, 300, 519])
def test_attention_finds_one_key_far_back_and_never_looks_ahead(dev, far):
    """Key ``far`` is aligned with the last queries (its score dominates); the key right after
    each query is aligned even more strongly and must stay invisible to it."""
    torch.manual_seed(2)
    L, Lq, H, G, D, E, bs = 520, 3, 4, 2, 8, 5, 16
    k, v = 0.1 * torch.randn(L, G, D), torch.randn(L, G, E)
    q = torch.randn(Lq, H, D)
    k[far] = 4.0 * q[-1].view(G, H // G, D).mean(1)
    for i in range(Lq - 1):                                   # the token after query i: a trap
        k[L - Lq + i + 1] = 9.0 * q[i].view(G, H // G, D).mean(1)
    sink, gate = torch.randn(H), torch.randn(Lq, H)
    want = orc.sink_attention(q.double(), k.double(), v.double(), 1.3, sink.double(), q_start=L - Lq)
    want = (want * torch.sigmoid(gate.double())[:, :, None]).float()
    kc, vc, table = _cache_from(k, v, bs)
    cu_q = torch.tensor([0, Lq], dtype=torch.int32)
    cu_k = torch.tensor([0, L], dtype=torch.int32)
    out = torch.zeros(Lq, H, E)
    if dev == "cpu":
        ops.sink_attention_prefill(q, kc, vc, cu_q, cu_k, table, 1.3, sink, gate, out)
    else:
        out = out.to(dev)
        pos = torch.arange(L - Lq, L, dtype=torch.int32)
        ops.sink_attention_step(*to(dev, q, kc, vc, table, torch.zeros(Lq, dtype=torch.int32), pos),
                                1.3, sink.to(dev), gate.to(dev), out)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-4, atol=1e-5)
    # the last query alone, as a decode row
    out1 = torch.zeros(1, H, E).to(dev)
    ops.sink_attention_decode(*to(dev, q[-1:], kc, vc, table, torch.tensor([L], dtype=torch.int32)),
                              1.3, sink.to(dev), gate[-1:].to(dev), out1)
    torch.testing.assert_close(out1.cpu(), want[-1:], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dev", DEVICES)
def test_sink_takes_weight_but_adds_nothing(dev):
    torch.manual_seed(3)
    L, H, G, D, E = 6, 2, 1, 4, 3
    k, v, q = torch.randn(L, G, D), torch.randn(L, G, E), torch.randn(1, H, D)
    kc, vc, table = _cache_from(k, v, 4)
    for s in (-50.0, 0.7, 12.0):
        sink = torch.tensor([s, -s])
        out = torch.zeros(1, H, E).to(dev)
        ops.sink_attention_decode(*to(dev, q, kc, vc, table, torch.tensor([L], dtype=torch.int32)),
                                  1.0, sink.to(dev), None, out)
        want = orc.sink_attention(q.double(), k.double(), v.double(), 1.0, sink.double(), q_start=L - 1)
        torch.testing.assert_close(out.cpu(), want.float(), rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_delta_rule_in_portions(dev, taps):
    """A sequence cut into portions of 1, 2, 1, 9 and 30 tokens (the first ones shorter than the
    convolution) next to a second one, state slots dirty at the start."""
    torch.manual_seed(4)
    H, G, D, E = 4, 2, 6, 10
    n = 43
    sizes = [G * D, G * D, H * E, H, H]
    proj = [torch.randn(n, sum(sizes)), torch.randn(n, sum(sizes))]
    conv_w = 0.6 * torch.randn(2 * G * D + H * E, taps)
    a_log, dt_bias = torch.randn(H) - 1, torch.randn(H)
    state = torch.randn(3, H, D, E).to(dev)
    conv = torch.randn(3, max(taps - 1, 0), 2 * G * D + H * E).to(dev)
    slots = torch.tensor([2, 0], dtype=torch.int32)
    want = []
    for p in proj:
        q, k, v, b, a = p.double().split(sizes, -1)
        cw = conv_w.double()
        q, _ = orc.short_conv(q, cw[:G * D], None)
        k, _ = orc.short_conv(k, cw[G * D:2 * G * D], None)
        v, _ = orc.short_conv(v, cw[2 * G * D:], None)
        q, k, v = orc.silu(q).view(n, G, D), orc.silu(k).view(n, G, D), orc.silu(v).view(n, H, E)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(b)
        g = torch.exp(-torch.exp(a_log.double()) * orc.softplus(a + dt_bias.double()))
        o, S = orc.gated_delta_rule(q.repeat_interleave(H // G, 1), k.repeat_interleave(H // G, 1), v, beta, g, None)
        want.append((o.float(), S.float()))
    got = [[], []]
    at = 0
    for cut in (1, 2, 1, 9, 30):
        rows = torch.cat([proj[0][at:at + cut], proj[1][at:at + cut]]).to(dev)
        T = 2 * cut
        cu_q = torch.tensor([0, cut, T], dtype=torch.int32).to(dev)
        pos = torch.cat([torch.arange(at, at + cut)] * 2).to(torch.int32).to(dev)
        row_seq = torch.tensor([0] * cut + [1] * cut, dtype=torch.int32).to(dev)
        q, k, v, b, a = rows.split(sizes, -1)
        prep = ops.delta_prepare(q.view(T, G, D), k.view(T, G, D), v.view(T, H, E), b, a, conv_w.to(dev),
                                 a_log.to(dev), dt_bias.to(dev), conv, cu_q, pos, slots.to(dev), row_seq=row_seq)
        o = ops.delta_scan(*prep, state, cu_q, pos, slots.to(dev)).cpu()
        got[0].append(o[:cut])
        got[1].append(o[cut:])
        at += cut
    for i in range(2):
        torch.testing.assert_close(torch.cat(got[i]), want[i][0], rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(state[int(slots[i])].cpu(), want[i][1], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dev", DEVICES)
def test_gated_head_norm(dev):
    torch.manual_seed(5)
    T, H, E = 5, 3, 7
    o, w, g = torch.randn(T, H, E), torch.randn(E), torch.randn(T, H * E)
    got = ops.gated_head_norm(*to(dev, o, w, g), 1e-3, torch.float32).cpu()
    want = orc.rms_unit(o.double(), 1e-3) * w.double() * orc.silu(g.double()).view(T, H, E)
    torch.testing.assert_close(got, want.float(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dev", DEVICES)
def test_router_keeps_groups_by_their_best_expert(dev):
    """Identity-like router: the logits are the input's first entries, set by hand."""
    NE, W = 8, 8
    wr = torch.eye(NE, W)
    z = torch.tensor([[5.0, 0.0, 0.1, 0.2, 4.0, 3.9, 3.8, 3.7],       # group 0 wins on one expert
                      [0.0, 0.1, 3.0, 0.2, 0.3, 9.0, 0.4, 0.5],       # groups 2 and 1 (of four)
                      [1.0, 2.0, 3.0, 4.0, 4.5, 0.0, 0.0, 0.0]])
    for top, groups, keep in ((2, 2, 1), (3, 4, 2), (4, 1, 1), (1, 8, 3)):
        dense = ops.grouped_route(z.to(dev), wr.to(dev), top, groups, keep).cpu()
        for t in range(z.shape[0]):
            ids, ws = orc.grouped_top_experts(z[t].double(), top, groups, keep)
            want = torch.zeros(NE)
            want[ids] = ws.float()
            torch.testing.assert_close(dense[t], want, rtol=1e-5, atol=1e-7)
    # the whole feed-forward against the oracle's
    torch.manual_seed(6)
    from minivllm_amd.layers.moe import GroupedRoutedExperts
    W, ff, NE = 12, 5, 6
    m = GroupedRoutedExperts(W, ff, NE, 2, 3, 2).to(dev)
    m.router.copy_(3 * torch.randn(NE, W)); m.up.copy_(torch.randn(NE * ff, W)); m.down.copy_(torch.randn(W, NE * ff))
    h = torch.randn(9, W)
    want = orc.routed_ffn(h.double(), m.router.cpu().double(), [m.up.cpu().double()[e * ff:(e + 1) * ff] for e in range(NE)],
                          [m.down.cpu().double()[:, e * ff:(e + 1) * ff] for e in range(NE)], 2, 3, 2)
    torch.testing.assert_close(m(h.to(dev)).cpu(), want.float(), rtol=1e-4, atol=1e-4)
