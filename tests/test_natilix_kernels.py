"""gfx950 kernels of the hybrid decoder (``ops.hip_hybrid``) against the plain PyTorch forms of
the same ops (``ops.torch_seqmix``) on CPU copies of the same inputs: bfloat16 and float32,
sizes that are not powers of two, several sequences per step, padding rows, portions shorter
than the convolution, state carried from one call to the next."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

gpu = torch.cuda.is_available()
if gpu:
    from minivllm_amd.ops import hip_hybrid as hk
from minivllm_amd.ops import torch_seqmix as ref

DTYPES = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_norms(dt):
    torch.manual_seed(0)
    T, W, V = 37, 200, 50
    table, aux = torch.randn(V, W).to(dt), torch.randn(12, W).to(dt)
    ids, rows = torch.randint(0, V, (T,), dtype=torch.int32), torch.randint(0, 12, (T,), dtype=torch.int32)
    x = ref.embed_sum(ids, rows, table, aux)
    xg = hk.embed_sum(*dev(ids, rows, table, aux))
    torch.testing.assert_close(xg.cpu(), x, rtol=0, atol=0)
    torch.testing.assert_close(hk.embed_sum(ids.cuda(), None, table.cuda(), None).cpu(),
                               ref.embed_sum(ids, None, table, None), rtol=0, atol=0)
    w, wb, wn = 0.2 * torch.randn(W), 0.2 * torch.randn(W), 0.2 * torch.randn(W)
    torch.testing.assert_close(hk.offset_rms_norm(xg, w.cuda(), 1e-5, dt).cpu().float(),
                               ref.offset_rms_norm(x, w, 1e-5, dt).float(), **tol(dt))
    y = torch.randn(T, W).to(dt)
    x2, xg2 = x.clone(), xg.clone()
    h = ref.post_norm_residual(y, wb, x2, 1e-5, wn, dt)
    hg = hk.post_norm_residual(y.cuda(), wb.cuda(), xg2, 1e-5, wn.cuda(), dt)
    torch.testing.assert_close(xg2.cpu(), x2, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(hg.cpu().float(), h.float(), **tol(dt))
    assert hk.post_norm_residual(y.cuda(), wb.cuda(), xg2, 1e-5, None, dt) is None


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_pair_rope_mix_store(dt, mode):
    torch.manual_seed(1)
    T, H, G, D, E, rot, bs, nb = 19, 6, 2, 24, 10, 16, 8, 7
    proj = torch.randn(T, H * D + G * D + G * E + H).to(dt)
    pos = torch.randint(0, 90, (T,), dtype=torch.int32)
    slots = torch.randperm(nb * bs)[:T].to(torch.int32)
    slots[3] = -1
    cs = ref.pair_cos_sin_table(rot, 128, 10000.0, dict(factor=4.0, low=1.0, high=4.0, original=64))
    vf = torch.randn(T, G, E).to(dt)
    lam = torch.tensor(0.3)
    out = {}
    for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: t.cuda())):
        p = to(proj.clone())
        q, k, v, _ = p.split([H * D, G * D, G * E, H], -1)
        kc, vc = to(torch.zeros(nb, bs, G, D, dtype=dt)), to(torch.zeros(nb, bs, G, E, dtype=dt))
        vfirst = to(vf.clone())
        mod.pair_rope_mix_store(q.view(T, H, D), k.view(T, G, D), v.view(T, G, E), to(pos), to(cs),
                                rot, vfirst, to(lam), mode, kc, vc, to(slots))
        out[name] = [t.cpu().float() for t in (p, kc, vc, vfirst)]
    for a, b in zip(out["gpu"], out["cpu"]):
        torch.testing.assert_close(a, b, **tol(dt))


def _paged(T_lens, bs, G, D, E, dt):
    nb = sum((n + bs - 1) // bs for n in T_lens) + 3
    perm = torch.randperm(nb).tolist()
    mb = max((n + bs - 1) // bs for n in T_lens)
    tables = torch.full((len(T_lens), mb), -1, dtype=torch.int32)
    for b, n in enumerate(T_lens):
        for j in range((n + bs - 1) // bs):
            tables[b, j] = perm.pop()
    return torch.randn(nb, bs, G, D).to(dt), torch.randn(nb, bs, G, E).to(dt), tables


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 64, 48), (5, 1, 20, 12), (8, 8, 16, 40), (12, 2, 32, 8)])
def test_sink_attention_decode_and_step(dt, H, G, D, E):
    torch.manual_seed(2)
    bs = 16
    lens = [1, 300, 0, 17, 257]
    kc, vc, tables = _paged(lens, bs, G, D, E, dt)
    B = len(lens)
    q = torch.randn(B, H, D).to(dt)
    gate, sink = torch.randn(B, H).to(dt), torch.randn(H)
    cl = torch.tensor(lens, dtype=torch.int32)
    o = ref.sink_attention_decode(q, kc, vc, tables, cl, 0.3, sink, gate, torch.zeros(B, H, E, dtype=dt))
    og = hk.sink_attention_decode(*dev(q, kc, vc, tables, cl), 0.3, sink.cuda(), gate.cuda(),
                                  torch.zeros(B, H, E, dtype=dt).cuda())
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))
    # prefill form: the last q_len rows of sequences 1, 3, 4, plus rows of no sequence
    qlens = [0, 40, 0, 17, 2]
    cu_q = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T = int(cu_q[-1]) + 3
    q = torch.randn(T, H, D).to(dt)
    gate = torch.randn(T, H).to(dt)
    row_seq = torch.full((T,), -1, dtype=torch.int32)
    pos = torch.zeros(T, dtype=torch.int32)
    for b, (n, L) in enumerate(zip(qlens, lens)):
        row_seq[cu_q[b]:cu_q[b + 1]] = b
        pos[cu_q[b]:cu_q[b + 1]] = torch.arange(L - n, L, dtype=torch.int32)
    o = ref.sink_attention_prefill(q, kc, vc, cu_q, cu_k, tables, 0.3, sink, gate,
                                   torch.zeros(T, H, E, dtype=dt))
    og = hk.sink_attention_step(*dev(q, kc, vc, tables, row_seq, pos), 0.3, sink.cuda(), gate.cuda(),
                                torch.zeros(T, H, E, dtype=dt).cuda())
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))
    # the prompt-portion entry point (matrix-core tiles where the head sizes have an instance)
    og = hk.sink_attention_prefill(*dev(q, kc, vc, cu_q, cu_k, tables), 0.3, sink.cuda(), gate.cuda(),
                                   torch.zeros(T, H, E, dtype=dt).cuda(), positions=pos.cuda(),
                                   max_q=max(qlens), row_seq=row_seq.cuda())
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))
    # ... and behind two sequences that are sliced off (a mixed step's decode riders)
    og = hk.sink_attention_prefill(*dev(q, kc, vc, cu_q[2:], cu_k[2:], tables[2:]), 0.3, sink.cuda(),
                                   gate.cuda(), torch.zeros(T, H, E, dtype=dt).cuda(),
                                   positions=pos.cuda(), max_q=max(qlens[2:]), row_seq=row_seq.cuda(),
                                   first_seq=2)
    lo = int(cu_q[2])
    torch.testing.assert_close(og.cpu().float()[lo:int(cu_q[-1])], o.float()[lo:int(cu_q[-1])], **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,E", [(2, 1, 128, 128), (4, 2, 64, 256), (2, 2, 200, 72), (2, 1, 260, 8)])
def test_sink_attention_prefill_long_portions(dt, H, G, D, E):
    """Portions longer than a workgroup's 128 queries, contexts that end inside a key tile,
    head sizes of every template instance and one (D > 256) that goes row by row."""
    torch.manual_seed(6)
    bs = 32
    lens, qlens = [700, 131, 33], [300, 131, 1]
    kc, vc, tables = _paged(lens, bs, G, D, E, dt)
    kc, vc = 0.3 * kc, vc
    cu_q = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T = int(cu_q[-1])
    q, gate, sink = torch.randn(T, H, D).to(dt), torch.randn(T, H).to(dt), torch.randn(H)
    row_seq = torch.zeros(T, dtype=torch.int32)
    pos = torch.zeros(T, dtype=torch.int32)
    for b, (n, L) in enumerate(zip(qlens, lens)):
        row_seq[cu_q[b]:cu_q[b + 1]] = b
        pos[cu_q[b]:cu_q[b + 1]] = torch.arange(L - n, L, dtype=torch.int32)
    o = ref.sink_attention_prefill(q, kc, vc, cu_q, cu_k, tables, D ** -0.5, sink, gate,
                                   torch.zeros(T, H, E, dtype=dt))
    og = hk.sink_attention_prefill(*dev(q, kc, vc, cu_q, cu_k, tables), D ** -0.5, sink.cuda(), gate.cuda(),
                                   torch.zeros(T, H, E, dtype=dt).cuda(), positions=pos.cuda(),
                                   max_q=max(qlens), row_seq=row_seq.cuda())
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,E,maxctx", [(4, 2, 128, 128, 2000), (8, 1, 64, 64, None), (2, 2, 256, 128, 300),
                                            (6, 2, 128, 64, 100000)])
def test_sink_attention_decode_split_contexts(dt, H, G, D, E, maxctx):
    """The head sizes of the split-context decode kernel: several splits, contexts shorter
    than a split, rows without a sequence, q rows strided as inside a projection output."""
    torch.manual_seed(7)
    bs = 16
    lens = [1, 1500, 0, 17, 257, 640]
    kc, vc, tables = _paged(lens, bs, G, D, E, dt)
    kc = 0.3 * kc
    B = len(lens)
    proj = torch.randn(B, H * D + 24).to(dt)
    gate, sink = torch.randn(B, H).to(dt), torch.randn(H)
    cl = torch.tensor(lens, dtype=torch.int32)
    o = ref.sink_attention_decode(proj[:, :H * D].view(B, H, D), kc, vc, tables, cl, D ** -0.5, sink, gate,
                                  torch.zeros(B, H, E, dtype=dt))
    pg = proj.cuda()
    og = hk.sink_attention_decode(pg[:, :H * D].view(B, H, D), *dev(kc, vc, tables, cl), D ** -0.5,
                                  sink.cuda(), gate.cuda(), torch.zeros(B, H, E, dtype=dt).cuda(), maxctx)
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))


def test_sink_decides_when_scores_are_low():
    """A large sink takes nearly all of the weight: the output shrinks towards zero."""
    H, G, D, E, bs = 2, 1, 8, 4, 4
    kc, vc, tables = _paged([9], bs, G, D, E, torch.float32)
    q = torch.randn(1, H, D)
    cl = torch.tensor([9], dtype=torch.int32)
    outs = []
    for s in (-30.0, 30.0):
        sink = torch.full((H,), s)
        outs.append(hk.sink_attention_decode(*dev(q, kc, vc, tables, cl), 1.0, sink.cuda(), None,
                                             torch.zeros(1, H, E).cuda()).cpu())
    assert outs[1].abs().max() < 1e-6 * max(outs[0].abs().max(), 1e-3) + 1e-5


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,E,taps", [(4, 2, 32, 48, 4), (3, 1, 20, 12, 2), (4, 4, 70, 40, 1),
                                          (2, 1, 128, 96, 5)])
def test_delta_prepare_and_scan(dt, H, G, D, E, taps):
    torch.manual_seed(3)
    slots_n = 6
    sizes = [G * D, G * D, H * E, H * E, H, H]
    conv_w = 0.5 * torch.randn(2 * G * D + H * E, taps)
    a_log, dt_bias = -1 + 0.5 * torch.randn(H), torch.randn(H)
    state0 = torch.randn(slots_n, H, D, E)
    conv0 = torch.randn(slots_n, max(taps - 1, 0), 2 * G * D + H * E)
    # three steps: prefill portions (one shorter than the convolution), then decode tokens
    steps = [([5, 1, 33], [0, 0, 7]), ([2, 40, 1], [5, 1, 40]), (None, [7, 41, 41])]
    slots = torch.tensor([4, 0, 2], dtype=torch.int32)
    res = {}
    for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: None if t is None else t.cuda())):
        torch.manual_seed(4)
        state, conv = to(state0.clone()), to(conv0.clone())
        outs = []
        for qlens, starts in steps:
            if qlens is None:
                T, cu_q, row_seq = 3, None, None
                pos = torch.tensor(starts, dtype=torch.int32)
                sl = slots
            else:
                qlens2 = qlens + [0]
                cu_q = torch.tensor([0] + list(torch.tensor(qlens2).cumsum(0)), dtype=torch.int32)
                T = int(cu_q[-1]) + 2
                row_seq = torch.full((T,), -1, dtype=torch.int32)
                pos = torch.zeros(T, dtype=torch.int32)
                for b, (n, s0) in enumerate(zip(qlens, starts)):
                    row_seq[cu_q[b]:cu_q[b + 1]] = b
                    pos[cu_q[b]:cu_q[b + 1]] = torch.arange(s0, s0 + n, dtype=torch.int32)
                sl = torch.cat([slots, torch.tensor([-1], dtype=torch.int32)])
            proj = to(torch.randn(T, sum(sizes)).to(dt))
            q, k, v, gate, b_, a_ = proj.split(sizes, -1)
            args = (q.view(T, G, D), k.view(T, G, D), v.view(T, H, E), b_, a_, to(conv_w),
                    to(a_log), to(dt_bias), conv, to(cu_q), to(pos), to(sl))
            prep = mod.delta_prepare(*args, to(row_seq)) if name == "gpu" else mod.delta_prepare(*args)
            o = mod.delta_scan(*prep, state, to(cu_q), to(pos), to(sl))
            valid = (row_seq >= 0) if row_seq is not None else torch.ones(T, dtype=torch.bool)
            outs += [t.cpu()[valid] for t in prep] + [o.cpu()[valid]]
        res[name] = outs + [state.cpu()[slots.long()], conv.cpu()[slots.long()]]
    t = tol(dt)
    for a, b in zip(res["gpu"], res["cpu"]):
        torch.testing.assert_close(a, b, rtol=max(t["rtol"], 1e-4), atol=max(t["atol"], 1e-4))


@pytest.mark.parametrize("dt", DTYPES)
def test_gated_head_norm_route_and_gelu(dt):
    torch.manual_seed(5)
    T, H, E = 9, 3, 20
    o, w, gate = torch.randn(T, H, E), 1 + 0.1 * torch.randn(E), torch.randn(T, H * E).to(dt)
    torch.testing.assert_close(hk.gated_head_norm(*dev(o, w, gate), 1e-5, dt).cpu().float(),
                               ref.gated_head_norm(o, w, gate, 1e-5, dt).float(), **tol(dt))
    for NE, top, groups, keep, W in ((8, 3, 2, 1, 64), (12, 3, 4, 2, 100), (6, 2, 1, 1, 33), (16, 1, 16, 3, 40)):
        h, wr = torch.randn(T, W).to(dt), torch.randn(NE, W)
        d = ref.grouped_route(h, wr, top, groups, keep)
        dg = hk.grouped_route(h.cuda(), wr.cuda(), top, groups, keep).cpu()
        assert ((d > 0) == (dg > 0)).all() and int((dg > 0).sum()) == T * top
        torch.testing.assert_close(dg, d, rtol=1e-4, atol=1e-6)
        ff = 10
        up = torch.randn(T, NE * ff).to(dt)
        torch.testing.assert_close(hk.gelu_route_scale(up.cuda(), dg.cuda(), ff, dt).cpu().float(),
                                   ref.gelu_route_scale(up, d, ff, dt).float(), **tol(dt))
