"""gfx950 kernels that the Pelenex family adds or extends (``ops.hip_hybrid``) against the plain
PyTorch forms of the same ops (``ops.torch_seqmix``) on CPU copies of the same inputs: bfloat16
and float32, sizes that are not powers of two, several sequences per step with unused rows, state
carried from one call to the next, windows whose edge falls inside a key tile."""
import pytest
import torch

pytestmark = pytest.mark.gpu

gpu = torch.cuda.is_available()
if gpu:
    from minivllm_amd.ops import hip_hybrid as hk
from minivllm_amd.ops import torch_seqmix as ref

DTYPES = [torch.float32, torch.bfloat16]


def tol(dt, f32=2e-5):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=f32, atol=f32)


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W,groups", [(200, 1), (192, 3), (96, 8), (2048, 2)])
def test_embedding_and_group_norms(dt, W, groups):
    torch.manual_seed(0)
    T, V = 37, 50
    table = torch.randn(V, W).to(dt)
    ids = torch.randint(0, V, (T,), dtype=torch.int32)
    pos = torch.randint(0, 5000, (T,), dtype=torch.int32)
    pos[0] = 0
    i = torch.arange(W // 2, dtype=torch.float64)
    inv = (10000.0 ** (-2.0 * i / W)).float()
    x = ref.embed_sinusoid(ids, pos, table, inv)
    xg = hk.embed_sinusoid(*dev(ids, pos, table, inv))
    torch.testing.assert_close(xg.cpu(), x, rtol=0, atol=2e-6)
    w = 1.0 + 0.2 * torch.randn(W)
    torch.testing.assert_close(hk.group_rms_norm(xg, w.cuda(), groups, 1e-5, dt).cpu().float(),
                               ref.group_rms_norm(x, w, groups, 1e-5, dt).float(), **tol(dt))
    wide = torch.randn(T, 3 * W).to(dt)
    y1, y2 = wide[:, :W], wide[:, 2 * W:]                      # rows of a wider tensor
    for ys in ([y1, y2], [y1], []):
        x2, xg2 = x.clone(), xg.clone()
        h = ref.residual_group_norm(x2, ys, w, groups, 1e-5, dt)
        wg = wide.cuda()
        hg = hk.residual_group_norm(xg2, [wg[:, :W], wg[:, 2 * W:]][:len(ys)], w.cuda(), groups, 1e-5, dt)
        torch.testing.assert_close(xg2.cpu(), x2, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(hg.cpu().float(), h.float(), **tol(dt))
    x2, xg2 = x.clone(), xg.clone()
    assert hk.residual_group_norm(xg2, [y1.cuda()], None, groups, 1e-5, dt) is None
    ref.residual_group_norm(x2, [y1], None, groups, 1e-5, dt)
    torch.testing.assert_close(xg2.cpu(), x2, rtol=1e-6, atol=1e-6)
    w2 = 1.0 + 0.2 * torch.randn(W)
    for parts in ([(y1, w), (y2, w2)], [(y2, w2)]):
        x2, xg2 = x.clone(), xg.clone()
        ref.add_normed_mean(x2, parts, 1e-5)
        hk.add_normed_mean(xg2, [(y.cuda(), v.cuda()) for y, v in parts], 1e-5)
        torch.testing.assert_close(xg2.cpu(), x2, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", DTYPES)
def test_unit_norm_store_cap_and_gated_activation(dt):
    torch.manual_seed(1)
    T, H, G, D, bs, nb = 19, 6, 2, 24, 8, 7
    proj = torch.randn(T, H * D + G * D + 5).to(dt)
    slots = torch.randperm(nb * bs)[:T].to(torch.int32)
    slots[3] = -1
    out = {}
    for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: t.cuda())):
        p = to(proj.clone())
        q, k, _ = p.split([H * D, G * D, 5], -1)
        kc, vc = to(torch.zeros(nb, bs, G, D, dtype=dt)), to(torch.zeros(nb, bs, G, D, dtype=dt))
        mod.unit_norm_store(q.view(T, H, D), k.view(T, G, D), 1e-5, kc, vc, to(slots))
        out[name] = [t.cpu().float() for t in (p, kc, vc)]
    for a, b in zip(out["gpu"], out["cpu"]):
        torch.testing.assert_close(a, b, **tol(dt))
    z = (20 * torch.randn(5, 70)).to(dt)
    torch.testing.assert_close(hk.tanh_cap_(z.clone().cuda(), 30.0).cpu().float(),
                               ref.tanh_cap_(z.clone(), 30.0).float(), **tol(dt))
    # routed gated activation: experts + a shared expert of another size, a dense layer (no router)
    for NE, ff, sff in ((5, 24, 40), (3, 7, 0), (0, 0, 56)):
        C = NE * ff + sff
        wide = torch.randn(T, 11 + 2 * C).to(dt)
        dense = None
        if NE:
            dense = torch.rand(T, NE) * (torch.rand(T, NE) < 0.4)
        a = ref.swiglu_route_scale(wide[:, 11:], dense, ff, sff, dt)
        ag = hk.swiglu_route_scale(wide.cuda()[:, 11:], None if dense is None else dense.cuda(), ff, sff, dt)
        torch.testing.assert_close(ag.cpu().float(), a.float(), **tol(dt))
        if NE:
            assert bool((ag.cpu()[:, :NE * ff].view(T, NE, ff)[dense == 0] == 0).all())


@pytest.mark.parametrize("dt", DTYPES)
def test_head_norm_and_sigmoid_router(dt):
    torch.manual_seed(2)
    T, H, E, W, NE = 23, 5, 12, 72, 11
    o = torch.randn(T, H, E)
    wide = torch.randn(T, H * E + 3).to(dt)
    for w, act in ((1 + 0.1 * torch.randn(H * E), "sigmoid"), (1 + 0.1 * torch.randn(E), "sigmoid"),
                   (1 + 0.1 * torch.randn(E), "silu")):
        y = ref.gated_head_norm(o, w, wide[:, 3:], 1e-5, dt, act)
        yg = hk.gated_head_norm(o.cuda(), w.cuda(), wide.cuda()[:, 3:], 1e-5, dt, act)
        torch.testing.assert_close(yg.cpu().float(), y.float(), **tol(dt))
    h = torch.randn(T, W).to(dt)
    rw = torch.randn(NE, W) * 0.3
    for top in (1, 3, NE):
        d = ref.grouped_route(h, rw, top, 1, 1, "sigmoid")
        dg = hk.grouped_route(h.cuda(), rw.cuda(), top, 1, 1, "sigmoid")
        assert bool(((dg.cpu() > 0) == (d > 0)).all())
        torch.testing.assert_close(dg.cpu(), d, rtol=1e-5, atol=1e-6)


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
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 64, 64), (5, 1, 20, 20), (4, 1, 96, 96), (8, 2, 128, 128)])
@pytest.mark.parametrize("window,keep", [(0, 0), (37, 5), (64, 0), (130, 40), (1, 3)])
def test_windowed_attention(dt, H, G, D, E, window, keep):
    """No sink, a window with kept first tokens and a distance penalty through all three kernels
    (rows, split decode, matrix-core tiles), against the CPU form."""
    torch.manual_seed(3)
    bs = 16
    lens = [1, 300, 0, 17, 257, 420]
    kc, vc, tables = _paged(lens, bs, G, D, E, dt)
    B = len(lens)
    q = torch.randn(B, H, D).to(dt)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])
    cl = torch.tensor(lens, dtype=torch.int32)
    opt = dict(window=window, keep_first=keep)
    o = ref.sink_attention_decode(q, kc, vc, tables, cl, 0.3, None, None, torch.zeros(B, H, E, dtype=dt),
                                  slopes=slopes, **opt)
    og = hk.sink_attention_decode(*dev(q, kc, vc, tables, cl), 0.3, None, None,
                                  torch.zeros(B, H, E, dtype=dt).cuda(), max(lens), slopes=slopes.cuda(), **opt)
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))
    qlens = [0, 140, 0, 17, 2, 333]
    cu_q = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T = int(cu_q[-1]) + 3
    q = torch.randn(T, H, D).to(dt)
    row_seq = torch.full((T,), -1, dtype=torch.int32)
    pos = torch.zeros(T, dtype=torch.int32)
    for b, (n, L) in enumerate(zip(qlens, lens)):
        row_seq[cu_q[b]:cu_q[b + 1]] = b
        pos[cu_q[b]:cu_q[b + 1]] = torch.arange(L - n, L, dtype=torch.int32)
    o = ref.sink_attention_prefill(q, kc, vc, cu_q, cu_k, tables, 0.3, None, None,
                                   torch.zeros(T, H, E, dtype=dt), slopes=slopes, **opt)
    og = hk.sink_attention_step(*dev(q, kc, vc, tables, row_seq, pos), 0.3, None, None,
                                torch.zeros(T, H, E, dtype=dt).cuda(), slopes=slopes.cuda(), **opt)
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))
    og = hk.sink_attention_prefill(*dev(q, kc, vc, cu_q, cu_k, tables), 0.3, None, None,
                                   torch.zeros(T, H, E, dtype=dt).cuda(), positions=pos.cuda(),
                                   max_q=max(qlens), row_seq=row_seq.cuda(), slopes=slopes.cuda(), **opt)
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))
    # with a sink as well: the options combine
    sink = torch.randn(H)
    o = ref.sink_attention_prefill(q, kc, vc, cu_q, cu_k, tables, 0.3, sink, None,
                                   torch.zeros(T, H, E, dtype=dt), **opt)
    og = hk.sink_attention_prefill(*dev(q, kc, vc, cu_q, cu_k, tables), 0.3, sink.cuda(), None,
                                   torch.zeros(T, H, E, dtype=dt).cuda(), positions=pos.cuda(),
                                   max_q=max(qlens), row_seq=row_seq.cuda(), **opt)
    torch.testing.assert_close(og.cpu().float(), o.float(), **tol(dt))


def _layout(lens, starts, slots):
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T = int(cu[-1])
    pos = torch.zeros(T, dtype=torch.int32)
    for b, (n, s) in enumerate(zip(lens, starts)):
        pos[cu[b]:cu[b + 1]] = torch.arange(s, s + n, dtype=torch.int32)
    return cu, pos, torch.tensor(slots, dtype=torch.int32), T


def _two_steps(run, S, lens1, lens2, slots):
    """A prefill-form step, then a second one that continues some sequences, then a decode-form
    step (one row per sequence); returns outputs and final states."""
    outs = []
    cu, pos, sl, T = _layout(lens1, [0] * len(lens1), slots)
    outs.append(run(T, cu, pos, sl, 0))
    cu, pos, sl, T = _layout(lens2, lens1, slots)
    outs.append(run(T, cu, pos, sl, 1))
    B = len(slots)
    pos = torch.tensor([a + b for a, b in zip(lens1, lens2)], dtype=torch.int32)
    outs.append(run(B, None, pos, sl, 2))
    return outs


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("lanes", ["4", "8", "16", ""])
@pytest.mark.parametrize("H,D,E", [(3, 48, 48), (2, 16, 80), (1, 130, 24), (4, 64, 64), (2, 32, 168)])
def test_mlstm_and_gla_scans(dt, H, D, E, lanes, monkeypatch):
    """``lanes``: lanes per state column of the scan kernel (empty: its own choice)."""
    monkeypatch.setenv("MINIVLLM_SCAN_LPC", lanes)
    torch.manual_seed(4)
    S = 5
    lens1, lens2, slots = [37, 1, 0, 20], [3, 18, 0, 1], [4, 0, -1, 2]
    n_in = 2 * H * D + H * E + 2 * H + H * D
    projs = [torch.randn(sum(l), n_in + 3).to(dt) for l in (lens1, lens2)] + [torch.randn(4, n_in + 3).to(dt)]
    for p in projs:
        p[:, 2 * H * D + H * E:2 * H * D + H * E + 2 * H] *= 6       # gates that reach the cap
    bi, bf, ab = torch.randn(H), 2 + torch.randn(H), torch.randn(H * D)
    Z = (E + 15) // 16             # copies of the normaliser and the running maximum per head
    init = [torch.randn(S, H, D, E), torch.randn(S, H, 1, D).expand(S, H, Z, D).contiguous(),
            torch.randn(S, H, 1).expand(S, H, Z).contiguous(), torch.randn(S, H, D, E)]
    res = {}
    for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: t.cuda())):
        st = [to(t.clone()) for t in init]

        def run(T, cu, pos, sl, step):
            p = to(projs[step])
            q, k, v, gi, gf, a = p[:, :n_in].split([H * D, H * D, H * E, H, H, H * D], -1)
            lay = (None if cu is None else to(cu), to(pos), to(sl))
            o1 = mod.mlstm_scan(q.view(-1, H, D), k.view(-1, H, D), v.view(-1, H, E), gi, gf, to(bi),
                                to(bf), 7.0, st[0], st[1], st[2], *lay)
            o2 = mod.gla_scan(q.view(-1, H, D), k.view(-1, H, D), v.view(-1, H, E), a.contiguous(),
                              to(ab), 4.0, st[3], *lay)
            return o1.cpu(), o2.cpu()
        res[name] = (_two_steps(run, S, lens1, lens2, slots), [s.cpu() for s in st])
    t = tol(dt, 1e-4)
    for (a1, a2), (b1, b2) in zip(res["gpu"][0], res["cpu"][0]):
        torch.testing.assert_close(a1, b1, **t)
        torch.testing.assert_close(a2, b2, **t)
    used = [s for s in slots if s >= 0]
    for a, b in zip(res["gpu"][1], res["cpu"][1]):
        torch.testing.assert_close(a[used], b[used], **t)
        other = [s for s in range(S) if s not in used]
        torch.testing.assert_close(a[other], b[other], rtol=0, atol=0)      # untouched slots


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("lanes", ["4", "8", "16"])
@pytest.mark.parametrize("H,G,D,E,taps", [(4, 2, 32, 32, 3), (2, 2, 24, 40, 4), (3, 1, 130, 16, 1)])
def test_channel_delta(dt, H, G, D, E, taps, lanes, monkeypatch):
    monkeypatch.setenv("MINIVLLM_SCAN_LPC", lanes)
    torch.manual_seed(5)
    S = 5
    lens1, lens2, slots = [37, 1, 0, 20], [3, 18, 0, 1], [4, 0, -1, 2]
    C = 2 * G * D + H * E
    n_in = C + H
    projs = [torch.randn(sum(l), n_in + 3).to(dt) for l in (lens1, lens2)] + [torch.randn(4, n_in + 3).to(dt)]
    arows = [torch.randn(p.shape[0], H * D).to(dt) for p in projs]
    conv_w, a_log, dtb = 0.5 * torch.randn(C, taps), -1 + 0.5 * torch.randn(H), torch.randn(H * D)
    init = [torch.randn(S, H, D, E), torch.randn(S, max(taps - 1, 0), C)]
    res = {}
    for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: t.cuda())):
        state, tail = to(init[0].clone()), to(init[1].clone())

        def run(T, cu, pos, sl, step):
            p = to(projs[step])
            q, k, v, b = p[:, :n_in].split([G * D, G * D, H * E, H], -1)
            lay = (None if cu is None else to(cu), to(pos), to(sl))
            rs = None
            if cu is not None:
                rs = torch.full((T,), -1, dtype=torch.int32)
                for i in range(len(sl)):
                    rs[cu[i]:cu[i + 1]] = i
                rs = to(rs)
            if name == "gpu":
                pre = mod.delta_prepare(q.view(-1, G, D), k.view(-1, G, D), v.view(-1, H, E), b,
                                        to(arows[step]), to(conv_w), to(a_log), to(dtb), tail, *lay, rs)
            else:
                pre = mod.delta_prepare(q.view(-1, G, D), k.view(-1, G, D), v.view(-1, H, E), b,
                                        to(arows[step]), to(conv_w), to(a_log), to(dtb), tail, *lay)
            assert pre[4].shape == (p.shape[0], H, D)
            o = mod.delta_scan(*pre, state, *lay)
            return (o.cpu(),) + tuple(x.cpu() for x in pre)
        res[name] = (_two_steps(run, S, lens1, lens2, slots), state.cpu(), tail.cpu())
    t = tol(dt, 1e-4)
    for step, (a, b) in enumerate(zip(res["gpu"][0], res["cpu"][0])):
        for x, y in zip(a, b):
            if step < 2:          # rows of the sequence without a slot are not computed
                cu = [0] + list(torch.tensor((lens1, lens2)[step]).cumsum(0))
                keep = torch.cat([torch.arange(cu[i], cu[i + 1]) for i in range(4) if slots[i] >= 0])
            else:
                keep = torch.tensor([i for i in range(4) if slots[i] >= 0])
            torch.testing.assert_close(x[keep], y[keep], **t)
    used = [s for s in slots if s >= 0]
    torch.testing.assert_close(res["gpu"][1][used], res["cpu"][1][used], **t)
    torch.testing.assert_close(res["gpu"][2][used], res["cpu"][2][used], **t)
