"""gfx950 kernels of the layer-list decoders (_k8sllm_hybrid) against the fp32 torch form of the
same op, bf16 and fp32 activations, at sizes that are not multiples of the kernels' tiles."""
import math

import pytest
import torch

from k8s_llm_monitor_amd.ops import hybrid as H

pytestmark = pytest.mark.gpu
DT = [torch.float32, torch.bfloat16]


def _tol(dt):
    return dict(rtol=2e-5, atol=2e-5) if dt == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def _g(seed=0):
    return torch.Generator().manual_seed(seed)


def _r(g, *shape, s=1.0, dt=torch.float32):
    return (torch.randn(*shape, generator=g) * s).to(dt)


def _i32(x):
    return torch.tensor(x, dtype=torch.int32)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("d", [72, 70, 2304])  # 8-wide vector path, scalar path, several trips per thread
def test_embed_pos_and_add_norm(dt, d):
    g = _g(1)
    V, T = 50, 7
    emb, pos = _r(g, V, d, dt=dt), _r(g, 40, d, dt=dt)
    ids, p = torch.randint(0, V, (T,), generator=g, dtype=torch.int32), torch.randint(0, 40, (T,), generator=g, dtype=torch.int32)
    src, prev = _i32([-1, 2, -1, 0, -1, -1, 1]), _i32([5, 6, 7])
    want = H.embed_pos(ids, p, emb, pos, src, prev)
    got = H.embed_pos(ids.cuda(), p.cuda(), emb.cuda(), pos.cuda(), src.cuda(), prev.cuda())
    assert torch.equal(got.cpu(), want)
    a, b, x0, vec, w = _r(g, T, d, dt=dt), _r(g, T, d), _r(g, T, d), _r(g, d), _r(g, d, s=0.2)
    for one_plus, adds, v in ((True, (a, b, x0), vec), (False, (a,), None), (True, (), None)):
        r_c, r_g = want.clone(), want.clone().cuda()
        y_c = H.add_norm(r_c, adds, v, w, 1e-5, one_plus, dt)
        y_g = H.add_norm(r_g, tuple(t.cuda() for t in adds), v.cuda() if v is not None else None, w.cuda(), 1e-5, one_plus, dt)
        torch.testing.assert_close(r_g.cpu(), r_c, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(y_g.cpu().float(), y_c.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
def test_gated_group_norm_and_swiglu(dt):
    g = _g(2)
    T, n, groups = 5, 96, 3
    y, proj, w = _r(g, T, n), _r(g, T, n + 40, dt=dt), _r(g, n, s=0.3) + 1
    want = H.gated_group_norm(y, proj, 8, w, 1e-5, groups, dt)
    got = H.gated_group_norm(y.cuda(), proj.cuda(), 8, w.cuda(), 1e-5, groups, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
    gu = _r(g, T, 2 * 37, dt=dt)
    torch.testing.assert_close(H.swiglu(gu.cuda()).cpu().float(), H.swiglu(gu).float(), **_tol(dt))


def _paged(g, dt, lens, Hq, G, dk, dv, nb=40, bs=16, shuffle=True):
    """Random q rows and a paged cache holding ``lens`` tokens per sequence on shuffled pages."""
    perm = torch.randperm(nb, generator=g).tolist() if shuffle else list(range(nb))
    W = max((n + bs - 1) // bs for n in lens)
    bt = torch.zeros(len(lens), W, dtype=torch.int32)
    kc, vc = _r(g, nb, bs, G * dk, dt=dt), _r(g, nb, G, dv, bs, dt=dt)
    for s, n in enumerate(lens):
        for j in range((n + bs - 1) // bs):
            bt[s, j] = perm.pop()
    return kc, vc, bt


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("window,sink", [(5, True), (0, True), (70, False), (16, True)])
def test_window_attention_kernels(dt, window, sink):
    g = _g(3)
    Hq, G, dk, dv = 6, 2, 24, 40
    ctx, new = [0, 37, 130], [9, 20, 3]
    lens = [c + n for c, n in zip(ctx, new)]
    kc, vc, bt = _paged(g, dt, lens, Hq, G, dk, dv)
    cu = _i32([0] + torch.tensor(new).cumsum(0).tolist())
    qkv = _r(g, sum(new), Hq * dk + G * (dk + dv), dt=dt)
    a = (Hq, G, dk, dv, 0.3, window, sink)
    want = H.window_attention_prefill(qkv, kc, vc, cu, _i32(ctx), bt, *a)
    got = H.window_attention_prefill(qkv.cuda(), kc.cuda(), vc.cuda(), cu.cuda(), _i32(ctx).cuda(), bt.cuda(), *a)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
    # decode: one query per sequence (plus a padding row of length 0)
    q1 = _r(g, 4, Hq * dk + G * (dk + dv), dt=dt)
    sl = _i32(lens + [0])
    bt4 = torch.cat([bt, torch.zeros(1, bt.shape[1], dtype=torch.int32)])
    want = H.window_attention_decode(q1, kc, vc, bt4, sl, *a)
    got = H.window_attention_decode(q1.cuda(), kc.cuda(), vc.cuda(), bt4.cuda(), sl.cuda(), *a)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
def test_qk_norm_cache(dt):
    g = _g(4)
    Hq, G, dk, dv, T = 3, 1, 20, 12, 6
    qkv = _r(g, T, Hq * dk + G * (dk + dv), dt=dt)
    qw, kw = _r(g, Hq * dk, s=0.3) + 1, _r(g, G * dk, s=0.3) + 1
    slots = _i32([17, 3, -1, 40, 41, 0])
    kc, vc = torch.zeros(4, 16, G * dk, dtype=dt), torch.zeros(4, G, dv, 16, dtype=dt)
    a_c, a_g = qkv.clone(), qkv.clone().cuda()
    kg, vg = kc.clone().cuda(), vc.clone().cuda()
    H.qk_norm_cache(a_c, qw, kw, 1e-5, Hq, G, dk, dv, kc, vc, slots)
    H.qk_norm_cache(a_g, qw.cuda(), kw.cuda(), 1e-5, Hq, G, dk, dv, kg, vg, slots.cuda())
    torch.testing.assert_close(a_g.cpu().float(), a_c.float(), **_tol(dt))
    torch.testing.assert_close(kg.cpu().float(), kc.float(), **_tol(dt))
    torch.testing.assert_close(vg.cpu().float(), vc.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("taps", [1, 2, 4])
@pytest.mark.parametrize("C,col0,pad", [(70, 9, 5), (72, 8, 8)])  # scalar path / 8 channels per thread
def test_conv_silu_with_state(dt, taps, C, col0, pad):
    g = _g(5)
    new, ctx, slot = [5, 1, 2, 3], [0, 4, 7, 0], [2, 0, -1, 3]
    T = sum(new)
    proj = _r(g, T, col0 + C + pad, dt=dt)
    cw, cb = _r(g, C, taps, s=0.5), _r(g, C, s=0.1)
    state = _r(g, 4, max(1, taps - 1), C, dt=dt)
    cu = _i32([0] + torch.tensor(new).cumsum(0).tolist())
    s_c, s_g = state.clone(), state.clone().cuda()
    want = H.conv_silu(proj, col0, C, cw, cb, s_c, cu, _i32(ctx), _i32(slot))
    got = H.conv_silu(proj.cuda(), col0, C, cw.cuda(), cb.cuda(), s_g, cu.cuda(), _i32(ctx).cuda(), _i32(slot).cuda())
    live = torch.tensor([r for s in range(4) if slot[s] >= 0 for r in range(int(cu[s]), int(cu[s + 1]))])
    torch.testing.assert_close(got.cpu().float()[live], want.float()[live], **_tol(dt))
    if taps > 1:
        torch.testing.assert_close(s_g.cpu().float(), s_c.float(), rtol=0, atol=0)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("nh,P,N,G", [(4, 24, 12, 2), (2, 80, 40, 1), (3, 16, 130, 3), (2, 20, 24, 2), (2, 40, 100, 1),
                                      (1, 8, 8, 1)])  # 2, 8, 32, 4, 16 lanes per value of p; state 8: the decode mapping only
def test_ssm_scan_with_state(dt, nh, P, N, G):
    g = _g(6)
    new, ctx, slot = [6, 1, 3, 40, 2], [0, 9, 2, 0, 1], [1, 3, 0, 2, -1]
    T = sum(new)
    inner = nh * P
    xbc = _r(g, T, inner + 2 * G * N, s=0.7, dt=dt)
    proj = _r(g, T, 11 + nh, dt=dt)
    dtb, alog, dsk = _r(g, nh, s=0.5) - 1, _r(g, nh, s=0.5) - 0.5, _r(g, nh) + 1
    state = _r(g, 4, nh, N, P)
    cu = _i32([0] + torch.tensor(new).cumsum(0).tolist())
    s_c, s_g = state.clone(), state.clone().cuda()
    want = H.ssm_scan(xbc, proj, 11, dtb, alog, dsk, s_c, cu, _i32(ctx), _i32(slot), nh, P, N, G)
    for mode in (1, 2):  # both lane mappings
        s_g = state.clone().cuda()
        got = H.ssm_scan(xbc.cuda(), proj.cuda(), 11, dtb.cuda(), alog.cuda(), dsk.cuda(), s_g, cu.cuda(),
                         _i32(ctx).cuda(), _i32(slot).cuda(), nh, P, N, G, mode=mode)
        torch.testing.assert_close(got.cpu(), want, rtol=2e-5, atol=2e-5)
        torch.testing.assert_close(s_g.cpu(), s_c, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("E,K,shared", [(5, 2, True), (12, 3, True), (24, 4, False), (70, 1, True)])
def test_router_and_experts(dt, E, K, shared):
    g = _g(7)
    T, d, ff = 45, 72, 40
    h = _r(g, T, d, dt=dt)
    wr, bias = _r(g, E + (1 if shared else 0), d, s=0.3), _r(g, E, s=0.3)
    ids_c, w_c, gate_c = H.moe_router(h, wr, bias, E, K)
    ids_g, w_g, gate_g = H.moe_router(h.cuda(), wr.cuda(), bias.cuda(), E, K)
    assert torch.equal(ids_g.cpu(), ids_c)
    torch.testing.assert_close(w_g.cpu(), w_c, rtol=1e-4, atol=1e-5)
    if shared:
        torch.testing.assert_close(gate_g.cpu(), gate_c, rtol=1e-4, atol=1e-5)
    w13, w2 = _r(g, E, 2 * ff, d, s=1 / math.sqrt(d), dt=dt), _r(g, E, d, ff, s=1 / math.sqrt(ff), dt=dt)
    sh = _r(g, T, d, dt=dt) if shared else None
    want = H.moe_experts(h, ids_c, w_c, w13, w2, sh, gate_c)
    got = H.moe_experts(h.cuda(), ids_g, w_g, w13.cuda(), w2.cuda(), sh.cuda() if shared else None, gate_g)
    torch.testing.assert_close(got.cpu(), want, **_tol(dt))


# ------------------------------------------------------------------ matrix-core / vector paths (bf16)

@pytest.mark.parametrize("dk,dv,Hq,G", [(64, 64, 4, 2), (128, 128, 2, 1), (64, 128, 3, 3), (128, 64, 8, 2)])
@pytest.mark.parametrize("window,sink", [(5, True), (16, True), (40, False), (0, True), (17, True)])
def test_window_prefill_mfma(dk, dv, Hq, G, window, sink):
    """Chunks that start inside a page, are shorter than a 16-row tile, or end one row into a tile;
    windows at, below and above the tile size."""
    g = _g(8)
    dt = torch.bfloat16
    ctx, new = [0, 40, 130, 7, 16, 3], [37, 5, 33, 1, 16, 150]
    lens = [c + n for c, n in zip(ctx, new)]
    kc, vc, bt = _paged(g, dt, lens, Hq, G, dk, dv)
    cu = _i32([0] + torch.tensor(new).cumsum(0).tolist())
    qkv = _r(g, sum(new), Hq * dk + G * (dk + dv), dt=dt)
    a = (Hq, G, dk, dv, 1.0 / math.sqrt(dk), window, sink)
    want = H.window_attention_prefill(qkv, kc, vc, cu, _i32(ctx), bt, *a)
    dev = [t.cuda() for t in (qkv, kc, vc, cu, _i32(ctx), bt)]
    for mode in (0, 1, 16, 32, 64):  # wave-per-row kernel, automatic, 16 / 32 / 64 query rows per wave
        got = H.window_attention_prefill(*dev, *a, mfma=mode)
        torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


def test_window_prefill_mfma_sees_exactly_the_window():
    """One key with a huge value: rows whose window holds it and rows whose window has just lost it."""
    g = _g(9)
    dt = torch.bfloat16
    Hq, G, dk, dv, window, n = 2, 1, 64, 64, 21, 90
    kc, vc, bt = _paged(g, dt, [n], Hq, G, dk, dv)
    far = 33
    vc.mul_(0.2)
    vc[int(bt[0, far // 16]), :, :, far % 16] = 100.0
    qkv = _r(g, n, Hq * dk + G * (dk + dv), dt=dt)
    a = (Hq, G, dk, dv, 0.01, window, True)
    dev = [t.cuda() for t in (qkv, kc, vc, _i32([0, n]), _i32([0]), bt)]
    for mode in (16, 32, 64):
        got = H.window_attention_prefill(*dev, *a, mfma=mode).cpu().float()
        seen = got.abs().amax(1) > 2.0  # the spike weighs at least 100 / (window + 1); everything else stays below 1
        assert seen.tolist() == [far <= r < far + window for r in range(n)]


@pytest.mark.parametrize("dk,dv,Hq,G", [(64, 64, 4, 2), (128, 128, 8, 1), (24, 16, 2, 2), (32, 256, 4, 4), (128, 64, 4, 1),
                                        (56, 40, 6, 3), (16, 200, 2, 1)])
@pytest.mark.parametrize("window", [7, 64, 100, 0])
def test_window_decode_vec(dk, dv, Hq, G, window):
    g = _g(10)
    dt = torch.bfloat16
    lens = [1, 64, 65, 200, 17]
    kc, vc, bt = _paged(g, dt, lens, Hq, G, dk, dv)
    q = _r(g, len(lens) + 1, Hq * dk + G * (dk + dv), dt=dt)
    sl = _i32(lens + [0])
    bt = torch.cat([bt, torch.zeros(1, bt.shape[1], dtype=torch.int32)])
    a = (Hq, G, dk, dv, 1.0 / math.sqrt(dk), window, True)
    want = H.window_attention_decode(q, kc, vc, bt, sl, *a)
    dev = [t.cuda() for t in (q, kc, vc, bt, sl)]
    torch.testing.assert_close(H.window_attention_decode(*dev, *a, vec=True).cpu().float(), want.float(), **_tol(dt))
    torch.testing.assert_close(H.window_attention_decode(*dev, *a, vec=False).cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("T,E,K,d,ff,il", [(45, 5, 2, 64, 96, False), (7, 8, 3, 128, 64, True), (300, 4, 2, 96, 128, True),
                                           (700, 4, 2, 128, 128, True), (1, 3, 1, 32, 32, False)])
def test_experts_matrix_core_paths(T, E, K, d, ff, il):
    """16-row matrix-core kernel (gathered rows, ragged last tiles, interleaved gate / up) and, from
    1024 sorted rows of an interleaved layer, the prefill tile GEMM."""
    from k8s_llm_monitor_amd import ops

    g = _g(11)
    dt = torch.bfloat16
    h = _r(g, T, d, dt=dt)
    wr, bias = _r(g, E + 1, d, s=0.3), _r(g, E, s=0.3)
    ids, w, gate = H.moe_router(h, wr, bias, E, K)
    w13 = _r(g, E, 2 * ff, d, s=1 / math.sqrt(d), dt=dt)
    w2 = _r(g, E, d, ff, s=1 / math.sqrt(ff), dt=dt)
    sh = _r(g, T, d, dt=dt)
    want = H.moe_experts(h, ids, w, w13, w2, sh, gate)
    w13g = torch.stack([ops.interleave_gate_up(x) for x in w13]).contiguous() if il else w13
    if il:  # the CPU form reads the interleaved layout too
        torch.testing.assert_close(H.moe_experts(h, ids, w, w13g, w2, sh, gate, il=True), want, rtol=1e-5, atol=1e-5)
    for mfma in (True, False):
        got = H.moe_experts(h.cuda(), ids.cuda(), w.cuda(), w13g.cuda(), w2.cuda(), sh.cuda(), gate.cuda(), il=il, mfma=mfma)
        torch.testing.assert_close(got.cpu(), want, **_tol(dt))


# ---------------------------------------------------------------- sequential-block designs' operators

@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("d", [72, 70, 2304])
def test_norm_shift_and_state(dt, d):
    """Segments of several rows and of one row, continuing from a slot or fresh, a padding segment;
    the state after the step; both steps of a prompt cut in two give the rows of the whole."""
    g = _g(11)
    T = 12
    x, w, mu = _r(g, T, d), _r(g, d, s=0.2) + 1, torch.rand(d, generator=g)
    cu, ctx, slot = _i32([0, 5, 6, 7, 12]), _i32([0, 9, 0, 3]), _i32([2, 0, -1, 1])
    st = _r(g, 4, d)
    for one_plus in (False, True):
        s_c, s_g = st.clone(), st.clone().cuda()
        want = H.norm_shift(x.clone(), (), w, 1e-6, one_plus, mu, s_c, cu, ctx, slot, dt)
        got = H.norm_shift(x.clone().cuda(), (), w.cuda(), 1e-6, one_plus, mu.cuda(), s_g, cu.cuda(), ctx.cuda(), slot.cuda(), dt)
        torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
        torch.testing.assert_close(s_g.cpu(), s_c, rtol=1e-5, atol=1e-5)
        assert torch.equal(s_g.cpu()[3], st[3])
    a = _r(g, T, d, dt=dt)
    s_c, s_g = st.clone(), st.clone().cuda()
    r_c, r_g = x.clone(), x.clone().cuda()
    want = H.norm_shift(r_c, (a,), w, 1e-6, False, mu, s_c, cu, ctx, slot, dt)
    got = H.norm_shift(r_g, (a.cuda(),), w.cuda(), 1e-6, False, mu.cuda(), s_g, cu.cuda(), ctx.cuda(), slot.cuda(), dt)
    torch.testing.assert_close(r_g.cpu(), r_c, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
    # one-row segments only (a decode step): no second launch
    cu1, ctx1, slot1 = torch.arange(T + 1, dtype=torch.int32), _i32([0, 3] * 6), _i32([2, 0, -1, 3, -1, 1] + [-1] * 6)
    s_c, s_g = st.clone(), st.clone().cuda()
    want = H.norm_shift(x.clone(), (), w, 1e-6, False, mu, s_c, cu1, ctx1, slot1, dt)
    got = H.norm_shift(x.clone().cuda(), (), w.cuda(), 1e-6, False, mu.cuda(), s_g, cu1.cuda(), ctx1.cuda(), slot1.cuda(), dt,
                       multi=False)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("n", [0, 1, 7])
def test_depth_mix(n):
    g = _g(12)
    T, d = 9, 36
    for add_dt in (None, torch.float32, torch.bfloat16):
        stack = _r(g, n + 3, T, d)
        coef = _r(g, n + 1)
        add = _r(g, T, d, dt=add_dt) if add_dt is not None else None
        s_c, s_g = stack.clone(), stack.clone().cuda()
        want = H.depth_mix(s_c, n, add, coef)
        got = H.depth_mix(s_g, n, add.cuda() if add is not None else None, coef.cuda())
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(s_g.cpu(), s_c, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh", "xielu"])
def test_activation(dt, kind):
    g = _g(13)
    for shape in ((5, 37), (3, 64)):
        x = _r(g, *shape, s=3.0, dt=dt)
        want = H.activation(x, kind, 0.6, 0.9)
        got = H.activation(x.cuda(), kind, 0.6, 0.9)
        torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("Q,R,dr,nf", [(20, 24, 8, 4), (300, 520, 6, 2), (8, 8, 2, 1)])
def test_latent_prep_and_queries(dt, Q, R, dr, nf):
    g = _g(14)
    T, H_, dn, bs, nb = 11, 3, 10, 16, 6
    proj = _r(g, T, Q + R + dr, dt=dt)
    qw, kw = _r(g, Q, s=0.2) + 1, _r(g, R, s=0.2) + 1
    pos = torch.randint(0, 3000, (T,), generator=g, dtype=torch.int32)
    freq = H.rotary_freq(1000.0, 2 * nf)
    slots = _i32([17, 3, -1, 95, 64, 0, 33, 34, 35, 80, 15])
    pitch = (R + dr + 31) // 32 * 32  # wider than the row: the tail stays zero
    kc, vc = torch.zeros(nb, bs, pitch, dtype=dt), torch.zeros(nb, 1, R, bs, dtype=dt)
    p_c, p_g, kg, vg = proj.clone(), proj.clone().cuda(), kc.clone().cuda(), vc.clone().cuda()
    H.latent_prep(p_c, Q, R, dr, qw, kw, 1e-6, pos, freq, kc, vc, slots)
    H.latent_prep(p_g, Q, R, dr, qw.cuda(), kw.cuda(), 1e-6, pos.cuda(), freq.cuda(), kg, vg, slots.cuda())
    tol = _tol(dt)
    torch.testing.assert_close(p_g.cpu().float(), p_c.float(), **tol)
    torch.testing.assert_close(kg.cpu().float(), kc.float(), **tol)
    torch.testing.assert_close(vg.cpu().float(), vc.float(), **tol)
    # a layer without key/value projection: only the query latent is normed
    p2 = proj[:, :Q].contiguous()
    p2c, p2g = p2.clone(), p2.clone().cuda()
    H.latent_prep(p2c, Q, R, dr, qw, None, 1e-6, pos, freq, None, None, None)
    H.latent_prep(p2g, Q, R, dr, qw.cuda(), None, 1e-6, pos.cuda(), freq.cuda(), None, None, None)
    torch.testing.assert_close(p2g.cpu().float(), p2c.float(), **tol)
    q, ql = _r(g, T, H_ * (dn + dr), dt=dt), _r(g, H_, T, R, dt=dt)
    for pt in (0, pitch):
        want = H.latent_queries(q, ql, H_, dn, dr, pos, freq, pt)
        got = H.latent_queries(q.cuda(), ql.cuda(), H_, dn, dr, pos.cuda(), freq.cuda(), pt)
        assert want.shape == (T, H_ * (pt or R + dr))
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol)
    assert float(kc[..., R + dr:].abs().max() if pitch > R + dr else 0.0) == 0.0
    assert float(kg[..., R + dr:].abs().max() if pitch > R + dr else 0.0) == 0.0


@pytest.mark.parametrize("dt", DT)
def test_attention_with_learned_sinks(dt):
    """Per-head sink logits in all four attention kernels (any-size and matrix-core prefill, any-size
    and vector decode) against the torch form."""
    g = _g(15)
    for Hq, G, dk, dv in ((8, 1, 104, 80), (4, 2, 64, 64), (3, 1, 20, 12)):
        lens, chunk = [50, 9, 33], [20, 9, 2]
        kc, vc, bt = _paged(g, dt, lens, Hq, G, dk, dv)
        sinks = _r(g, Hq, s=2.0)
        T = sum(chunk)
        qkv = _r(g, T, Hq * dk, s=0.3, dt=dt)
        cu = _i32([0, 20, 29, 31])
        ctx = _i32([n - c for n, c in zip(lens, chunk)])
        a = (Hq, G, dk, dv, 0.2, 24, True)
        want = H.window_attention_prefill(qkv, kc, vc, cu, ctx, bt, *a, sinks=sinks)
        base = H.window_attention_prefill(qkv, kc, vc, cu, ctx, bt, *a)
        assert float((want.float() - base.float()).abs().max()) > 1e-2  # the sinks are not a no-op
        dev = [t.cuda() for t in (qkv, kc, vc, cu, ctx, bt)]
        for mode in (1, 0):
            got = H.window_attention_prefill(*dev, *a, mfma=mode, sinks=sinks.cuda())
            torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
        q1 = _r(g, 3, Hq * dk, s=0.3, dt=dt)
        sl = _i32(lens)
        want = H.window_attention_decode(q1, kc, vc, bt, sl, *a, sinks=sinks)
        for vec in (True, False):
            got = H.window_attention_decode(q1.cuda(), kc.cuda(), vc.cuda(), bt.cuda(), sl.cuda(), *a, vec=vec, sinks=sinks.cuda())
            torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
def test_router_over_all_and_gelu_experts(dt):
    g = _g(16)
    T, d, E, K, ff = 37, 64, 6, 3, 48
    h = _r(g, T, d, dt=dt)
    wr = _r(g, E, d, s=0.3)
    ids_c, w_c, _ = H.moe_router(h, wr, None, E, K, over_all=True)
    ids_g, w_g, gate = H.moe_router(h.cuda(), wr.cuda(), None, E, K, over_all=True)
    assert gate is None and torch.equal(ids_g.cpu(), ids_c)
    torch.testing.assert_close(w_g.cpu(), w_c, rtol=1e-5, atol=1e-6)
    assert float(w_c.sum(-1).max()) < 1.0
    w1, w2 = _r(g, E, ff, d, s=d ** -0.5, dt=dt), _r(g, E, d, ff, s=ff ** -0.5, dt=dt)
    shared = _r(g, T, d, dt=dt)
    for sh in (None, shared):
        want = H.moe_experts(h, ids_c, w_c, w1, w2, sh, None, act="gelu")
        for mfma in (True, False):
            got = H.moe_experts(h.cuda(), ids_g, w_g, w1.cuda(), w2.cuda(), sh.cuda() if sh is not None else None, None,
                                act="gelu", mfma=mfma)
            torch.testing.assert_close(got.cpu(), want, **_tol(dt))


@pytest.mark.parametrize("Hq,pitch,dv", [(8, 128, 112), (16, 320, 256), (20, 64, 48), (3, 96, 16), (1, 32, 32)])
@pytest.mark.parametrize("window", [24, 0, 300])
def test_latent_attention_matrix_core(Hq, pitch, dv, window):
    """The head-packed matrix-core kernel (one wave per row, two rows per wave, the window split
    over four or eight waves, and the LDS-staged kernel of large steps)
    against the torch form: prompt chunks with context, single rows, padding rows, partial head groups."""
    dt = torch.bfloat16
    g = _g(17)
    lens, chunk = [350, 9, 33, 70], [20, 9, 2, 70]
    kc, vc, bt = _paged(g, dt, lens, Hq, 1, pitch, dv, nb=60)
    sinks = _r(g, Hq, s=1.5)
    T = sum(chunk)
    qa = _r(g, T, Hq * pitch, s=0.25, dt=dt)
    cu = _i32([0, 20, 29, 31, 101])
    ctx = _i32([n - c for n, c in zip(lens, chunk)])
    want = H.latent_attention(qa, kc, vc, bt, Hq, 0.2, window, sinks, cu=cu, ctx=ctx)
    dev = lambda *ts: [t.cuda() for t in ts]  # noqa: E731
    for split in (1, 2, 4, 8, 32, 33, 0):
        got = H.latent_attention(*dev(qa, kc, vc, bt), Hq, 0.2, window, sinks.cuda(), cu=cu.cuda(), ctx=ctx.cuda(),
                                 split=split)
        torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
    q1 = _r(g, 5, Hq * pitch, s=0.25, dt=dt)
    sl = _i32(lens + [0])  # the last row is a padding row
    bt5 = torch.cat([bt, bt[:1]])
    want = H.latent_attention(q1, kc, vc, bt5, Hq, 0.2, window, sinks, seq_lens=sl)
    for split in (1, 4, 8, 0):
        got = H.latent_attention(*dev(q1, kc, vc, bt5), Hq, 0.2, window, sinks.cuda(), seq_lens=sl.cuda(), split=split)
        torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
        assert float(got[4].abs().max()) == 0.0


def test_gelu_experts_on_the_tile_gemm():
    """Widths that are multiples of 256 and a large step: the ungated experts go through the
    prefill tile GEMM and agree with the 16-row kernel and the torch form."""
    dt = torch.bfloat16
    g = _g(18)
    T, d, E, K, ff = 700, 256, 4, 2, 512  # 1400 routed rows
    h = _r(g, T, d, dt=dt)
    wr = _r(g, E, d, s=0.3)
    ids, wts, _ = H.moe_router(h, wr, None, E, K, over_all=True)
    w1, w2 = _r(g, E, ff, d, s=d ** -0.5, dt=dt), _r(g, E, d, ff, s=ff ** -0.5, dt=dt)
    want = H.moe_experts(h, ids, wts, w1, w2, None, None, act="gelu")
    got = H.moe_experts(h.cuda(), ids.cuda(), wts.cuda(), w1.cuda(), w2.cuda(), None, None, act="gelu")
    torch.testing.assert_close(got.cpu(), want, **_tol(dt))
