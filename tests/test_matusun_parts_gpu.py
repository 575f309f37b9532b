"""The kernels that the Matusun design added, each alone, against the plain functions of
tests/plain_matusun.py or a few lines of float64 arithmetic: odd sizes, sequences cut at every kind
of place, state slots in any order and used again, keys just inside and just outside a window in
prompts and in decoding, routers with experts that return their input."""
import pytest
import torch

import plain_matusun as pm

pytestmark = pytest.mark.gpu


def dev(t, dtype=torch.float32):
    return t.to("cuda", dtype).contiguous()


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# ---- hyper-connections -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,H", [(1, 40), (2, 64), (3, 100), (4, 520), (7, 33), (16, 24)])
def test_streams_update_and_read_out(gpu_device, dtype, S, H):
    """The update behind a sublayer and the read-out with its norm, together and each alone, with
    learned coefficients and with none."""
    from pytriton_llama_amd import ops
    torch.manual_seed(S * 100 + H)
    T, eps = 19, 1e-5
    x = torch.randn(T, S, H, dtype=torch.float64)
    y = torch.randn(T, H, dtype=torch.float64)
    if dtype == torch.bfloat16:
        y = y.bfloat16().double()
    mix, outc, inc = (torch.randn(S, S, dtype=torch.float64), torch.randn(S, dtype=torch.float64),
                      torch.randn(S, dtype=torch.float64))
    nw = 1 + 0.2 * torch.randn(H, dtype=torch.float64)
    new = torch.einsum("sr,tsh->trh", mix, x) + outc[None, :, None] * y[:, None, :]
    read = pm.rms(torch.einsum("s,tsh->th", inc, new), eps) * nw
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    # both halves in one kernel
    st = dev(x.reshape(T, S * H))
    out = ops.hyper_mix(st, S, dev(y, dtype), dev(mix), dev(outc), dev(inc), dev(nw), eps, dtype)
    assert float((st.double().cpu().view(T, S, H) - new).abs().max()) < 2e-5 * float(new.abs().max())
    assert float((out.double().cpu() - read).abs().max()) < tol * float(read.abs().max())
    # the update alone, then the read-out alone
    st = dev(x.reshape(T, S * H))
    assert ops.hyper_mix(st, S, dev(y, dtype), dev(mix), dev(outc)) is None
    assert float((st.double().cpu().view(T, S, H) - new).abs().max()) < 2e-5 * float(new.abs().max())
    out = ops.hyper_mix(st, S, None, None, None, dev(inc), dev(nw), eps, dtype)
    assert float((out.double().cpu() - read).abs().max()) < tol * float(read.abs().max())
    # no coefficients: every stream takes y, the read-out is the sum of the streams
    st = dev(x.reshape(T, S * H))
    out = ops.hyper_mix(st, S, dev(y, dtype), None, None, None, dev(nw), eps, dtype)
    plain = x + y[:, None, :]
    assert float((st.double().cpu().view(T, S, H) - plain).abs().max()) < 2e-5 * float(plain.abs().max())
    want = pm.rms(plain.sum(1), eps) * nw
    assert float((out.double().cpu() - want).abs().max()) < tol * float(want.abs().max())


def test_embedding_written_once_a_stream(gpu_device):
    from pytriton_llama_amd import ops
    table = torch.randn(50, 24)
    ids = torch.randint(0, 50, (13,))
    out = ops.embedding_scaled(dev(table), i32(ids.tolist()), 1.0, 3).cpu()
    assert torch.equal(out.view(13, 3, 24), table[ids][:, None, :].expand(13, 3, 24))


# ---- the selective scan --------------------------------------------------------------------------
def cut(total, sizes):
    out, lo, k = [], 0, 0
    while lo < total:
        hi = min(total, lo + sizes[k % len(sizes)])
        out.append((lo, hi))
        lo, k = hi, k + 1
    return out


@pytest.mark.parametrize("C,N,R,taps", [(16, 16, 4, 4), (40, 8, 3, 3), (50, 20, 5, 1), (33, 40, 2, 2), (24, 130, 7, 4), (20, 8, 3, 9),
                                        (130, 12, 20, 5)])
def test_selective_scan_in_portions_and_batches(gpu_device, C, N, R, taps):
    """Three sequences advanced together in portions of changing sizes (down to one token, their
    ends inside and outside the 16-token chunks of the kernel), in state slots that are out of
    order, against the recurrence written out; then the slots are cleared and used again."""
    from pytriton_llama_amd import ops
    torch.manual_seed(C + N)
    lens = [75, 21, 40]
    slots = [2, 0, 3]
    f64 = torch.float64
    cw, cb = 0.5 * torch.randn(C, taps, dtype=f64), 0.1 * torch.randn(C, dtype=f64)
    w_dt, dt_b = torch.randn(C, R, dtype=f64) / R ** 0.5, torch.rand(C, dtype=f64) * 3 - 4
    A_log, D = torch.rand(C, N, dtype=f64) * 2.5 - 1, torch.randn(C, dtype=f64)
    pad = 3
    ps = [torch.randn(n, pad + 2 * C + 2, dtype=f64) for n in lens]       # u at pad, z behind it
    rs = [torch.randn(n, R + 2 * N + 1, dtype=f64) for n in lens]         # r | B | C
    want = []
    for p, r in zip(ps, rs):
        u = pm.silu(pm.causal_conv(p[:, pad:pad + C], cw, cb))
        dt = pm.softplus(r[:, :R] @ w_dt.T + dt_b)
        y = pm.selective_scan(u, dt, -torch.exp(A_log), r[:, R:R + N], r[:, R + N:R + 2 * N], D)
        want.append(y * pm.silu(p[:, pad + C:pad + 2 * C]))
    tail_off = C * N
    state = torch.randn(5, ops.selective_state_floats(C, N, taps), device="cuda")     # slots hold rubbish
    args = [dev(t) for t in (cw, cb, w_dt, dt_b, A_log, D)]
    for sizes in ((7, 1, 16, 2, 33, 1, 1, 5), (100,), (1,)):
        for s in slots:
            state[s].zero_()
        got = [torch.zeros(n, C, dtype=f64) for n in lens]
        cuts = [cut(n, sizes[i:] + sizes[:i]) for i, n in enumerate(lens)]
        for step in range(max(len(c) for c in cuts)):
            live = [i for i in range(3) if step < len(cuts[i])]
            rows_p = torch.cat([ps[i][cuts[i][step][0]:cuts[i][step][1]] for i in live])
            rows_r = torch.cat([rs[i][cuts[i][step][0]:cuts[i][step][1]] for i in live])
            qlens = [cuts[i][step][1] - cuts[i][step][0] for i in live]
            q_start = i32([0] + torch.tensor(qlens).cumsum(0).tolist())
            sl = i32([slots[i] for i in live])
            p_dev, r_dev = dev(rows_p), dev(rows_r)
            u, _ = ops.selective_conv(p_dev, pad, args[0], args[1], state, tail_off, q_start, sl, max(qlens))
            if taps > 1:
                ops.conv_tail_update(p_dev, pad, C, taps, state, tail_off, q_start, sl)
            y = ops.selective_scan(u, p_dev, pad + C, r_dev, R, R, R + N, args[2], args[3], args[4], args[5],
                                   state, q_start, sl, torch.float32).double().cpu()
            at = 0
            for i, n in zip(live, qlens):
                got[i][cuts[i][step][0]:cuts[i][step][1]] = y[at:at + n]
                at += n
        for g, w in zip(got, want):
            assert float((g - w).abs().max()) < 3e-5 * float(w.abs().max()), sizes


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,N,R,taps,seg", [(64, 16, 4, 4, 16), (40, 8, 3, 3, 32), (70, 20, 5, 2, 0), (130, 32, 9, 1, 64),
                                            (33, 5, 2, 3, 16), (24, 12, 40, 4, 0)])
def test_selective_scan_of_long_portions_in_segments(gpu_device, C, N, R, taps, seg, out_dtype):
    """Sequences of unequal lengths whose long portions are walked in segments side by side
    (portions that end inside a segment, at its end and one token behind it; a sequence of one
    token beside them; short portions of the same sequences through the chain before and after),
    against the recurrence written out; the state that the segments leave is the one that single
    tokens go on from."""
    from pytriton_llama_amd import ops
    torch.manual_seed(C * N + R)
    lens = [333, 1, 129, 200]
    slots = [1, 4, 0, 2]
    f64 = torch.float64
    cw, cb = 0.5 * torch.randn(C, taps, dtype=f64), 0.1 * torch.randn(C, dtype=f64)
    w_dt, dt_b = torch.randn(C, R, dtype=f64) / R ** 0.5, torch.rand(C, dtype=f64) * 3 - 4
    A_log, D = torch.rand(C, N, dtype=f64) * 2.5 - 1, torch.randn(C, dtype=f64)
    ps = [torch.randn(n, 2 * C, dtype=f64) for n in lens]
    rs = [torch.randn(n, R + 2 * N, dtype=f64) for n in lens]
    want = []
    for p, r in zip(ps, rs):
        u = pm.silu(pm.causal_conv(p[:, :C], cw, cb))
        dt = pm.softplus(r[:, :R] @ w_dt.T + dt_b)
        y = pm.selective_scan(u, dt, -torch.exp(A_log), r[:, R:R + N], r[:, R + N:R + 2 * N], D)
        want.append(y * pm.silu(p[:, C:]))
    tail_off = C * N
    state = torch.randn(5, ops.selective_state_floats(C, N, taps), device="cuda")
    args = [dev(t) for t in (cw, cb, w_dt, dt_b, A_log, D)]
    tol = 3e-5 if out_dtype == torch.float32 else 1e-2
    for sizes in ((400,), (3, 64, 1, 65, 2, 128, 1, 1, 100), (96, 1, 97)):
        for s_ in slots:
            state[s_].zero_()
        got = [torch.zeros(n, C, dtype=f64) for n in lens]
        cuts = [cut(n, sizes[i:] + sizes[:i]) for i, n in enumerate(lens)]
        for step in range(max(len(c) for c in cuts)):
            live = [i for i in range(len(lens)) if step < len(cuts[i])]
            rows_p = torch.cat([ps[i][cuts[i][step][0]:cuts[i][step][1]] for i in live])
            rows_r = torch.cat([rs[i][cuts[i][step][0]:cuts[i][step][1]] for i in live])
            qlens = [cuts[i][step][1] - cuts[i][step][0] for i in live]
            q_start = i32([0] + torch.tensor(qlens).cumsum(0).tolist())
            sl = i32([slots[i] for i in live])
            p_dev, r_dev = dev(rows_p), dev(rows_r)
            u, _ = ops.selective_conv(p_dev, 0, args[0], args[1], state, tail_off, q_start, sl, max(qlens))
            if taps > 1:
                ops.conv_tail_update(p_dev, 0, C, taps, state, tail_off, q_start, sl)
            y = ops.selective_scan(u, p_dev, C, r_dev, R, R, R + N, args[2], args[3], args[4], args[5],
                                   state, q_start, sl, out_dtype, max(qlens), seg).double().cpu()
            at = 0
            for i, n in zip(live, qlens):
                got[i][cuts[i][step][0]:cuts[i][step][1]] = y[at:at + n]
                at += n
        for g, w in zip(got, want):
            assert float((g - w).abs().max()) < tol * float(w.abs().max()), sizes


def test_segment_length_fills_the_chip():
    from pytriton_llama_amd import ops
    assert ops.selective_segment(1, 2048, 4096) == 32
    assert ops.selective_segment(8, 2048, 4096) == 256
    assert ops.selective_segment(1, 64, 64) == 16
    assert ops.selective_segment(1, 1 << 20, 8192) == 256


# ---- the router and the experts -----------------------------------------------------------------
@pytest.mark.parametrize("E,ident,top,shared", [(5, 2, 3, True), (4, 0, 1, False), (2, 1, 3, True), (70, 3, 4, False),
                                                (1, 1, 1, False)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_softmax_router_with_correction_and_experts_that_return_their_input(gpu_device, dtype, E, ident, top, shared):
    from pytriton_llama_amd.parts import build_part
    torch.manual_seed(E * 10 + top)
    W, I, T, scale = 48, 40, 37, 1.7
    sh = build_part("feed_forward", "mlp", hidden_size=W, intermediate_size=56) if shared else None
    part = build_part("feed_forward", "routed_experts", hidden_size=W, intermediate_size=I, num_experts=E, top=top,
                      activation="relu2", weight_on_input=False, renormalize=True, renorm_eps=1e-20,
                      route_scale=scale, score="softmax", correction_name="correction", identity=ident,
                      shared=sh, shared_gate=False)
    w = {}
    for src in part.param_sources():
        if src.name == "correction":
            w[src.name] = 0.05 * torch.randn(src.shape)
        elif src.name == "router":
            w[src.name] = torch.randn(src.shape)
        else:
            w[src.name] = 0.2 * torch.randn(src.shape)
        if src.kind == "matrix" and dtype == torch.bfloat16:
            w[src.name] = w[src.name].bfloat16().float()
    part.load(w, dtype, "cuda")
    h = torch.randn(T, W)
    if dtype == torch.bfloat16:
        h = h.bfloat16().float()
    got = part.forward(dev(h, dtype)).double().cpu()
    mlp = {"router": {"experts": E, "identity": ident, "top": top, "scale": scale}, "shared": {"ff": 56} if shared else None}
    w64 = {k: v.double() for k, v in w.items()}
    pm.ROUTER_MARGINS = []
    try:
        want = pm.routed_mlp(h.double(), mlp, w64)
        close = pm.ROUTER_MARGINS[0]
    finally:
        pm.ROUTER_MARGINS = None
    err = (got - want).abs().amax(-1) / want.abs().max()
    if dtype == torch.bfloat16:
        err = err[~close]
    assert float(err.max()) < (2e-5 if dtype == torch.float32 else 2e-2)
    # the routing itself: experts and weights
    from pytriton_llama_amd import ops
    logits = (h.double() @ w64["router"].T).float()
    r = ops.moe_route(dev(logits), E, top, 0, True, ops.SCORE_SOFTMAX, dev(w["correction"]), ident, 1e-20, scale)
    idx, wgt, _ = pm.route(h.double(), w64["router"], w64["correction"], top, scale)
    mine = r.idx.view(T, top).cpu()
    assert torch.equal(torch.where(mine < 0, -1, mine).sort(-1).values,
                       torch.where(idx >= E, -1, idx).int().sort(-1).values)
    assert float((r.wgt.view(T, top).cpu().double().sum(-1) - wgt.sum(-1)).abs().max()) < 1e-5
    if ident:
        want_ident = torch.where(idx >= E, wgt, torch.zeros_like(wgt)).sum(-1)
        assert float((r.ident.cpu().double() - want_ident).abs().max()) < 1e-5
    else:
        assert r.ident is None


def test_sigmoid_router_is_what_it_was(gpu_device):
    """The router of the gated experts (sigmoid scores, no correction, weights without a
    constant): chosen by the largest logits, ties to the lower index, with and without the
    division by the sum."""
    from pytriton_llama_amd import ops
    torch.manual_seed(2)
    T, E, top = 29, 9, 3
    z = torch.randn(T, E + 1)
    z[3, 2] = z[3, 5] = z[3].max() + 1           # a tie: the lower index first
    for renorm in (False, True):
        r = ops.moe_route(dev(z), E, top, 1, renorm)
        s = torch.sigmoid(z[:, :E].double())
        order = torch.sort(z[:, :E], dim=-1, descending=True, stable=True).indices[:, :top]
        assert torch.equal(r.idx.view(T, top).cpu().long(), order)
        w = torch.gather(s, 1, order)
        if renorm:
            w = w / w.sum(-1, keepdim=True)
        assert float((r.wgt.view(T, top).cpu().double() - w).abs().max()) < 1e-6
        assert float((r.extra.cpu().double()[:, 0] - torch.sigmoid(z[:, E].double())).abs().max()) < 1e-6


# ---- windows in the attention kernels -----------------------------------------------------------
def _windowed(q, k, v, n, ql, window, scale, H, G):
    out = torch.zeros(ql, H, v.shape[-1], dtype=torch.float64)
    pos = torch.arange(n - ql, n)[:, None]
    j = torch.arange(n)[None, :]
    vis = (j <= pos) & (pos - j < window)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        out[:, h] = torch.softmax(s.masked_fill(~vis, float("-inf")), -1) @ v[:, g]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,Dk,Dv,window,P", [(4, 2, 32, 64, 33, 16), (2, 1, 16, 48, 24, 8), (3, 3, 20, 12, 7, 4),
                                                (4, 4, 64, 32, 100, 16), (2, 2, 32, 32, 1, 8)])
def test_keys_just_inside_and_just_outside_a_window(gpu_device, dtype, H, G, Dk, Dv, window, P):
    """A portion of a prompt behind a cached prefix and a single decoded token, through every
    kernel that takes the sizes. The key at the window's first place (i - window + 1) and the one
    in front of it (i - window) are made to stand out for the last query of each sequence: the
    first must get nearly all the weight, the second none. Pages that lie wholly in front of the
    windows are not there (their table entries are -1)."""
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.engine.batch import work_items
    torch.manual_seed(window)
    pages, scale = 128, 0.3
    lens, qlens = [150, 205], [40, 1]
    order = torch.randperm(pages).tolist()
    k_pool = torch.randn(pages, G, P, Dk, dtype=torch.float64) * 5
    v_pool = torch.randn(pages, G, P, Dv, dtype=torch.float64) * 5
    bt = torch.full((2, -(-max(lens) // P)), -1, dtype=torch.int32)
    qs, want, at = [], [], 0
    for r, (n, ql) in enumerate(zip(lens, qlens)):
        k = torch.randn(n, G, Dk, dtype=torch.float64)
        v = torch.randn(n, G, Dv, dtype=torch.float64)
        q = torch.randn(ql, H, Dk, dtype=torch.float64)
        inside, outside = n - 1 - window + 1, n - 1 - window
        k[inside] *= 3.0
        q[-1, 0] = k[inside, 0] * 2.0
        if outside >= 0:
            k[outside] = k[inside] * 1.5            # would win if it were seen
        if dtype == torch.bfloat16:
            q, k, v = (t.bfloat16().double() for t in (q, k, v))
        out = _windowed(q, k, v, n, ql, window, scale, H, G)
        if window > 1:                               # the last query's first head reads the edge key
            assert float((out[-1, 0] - v[inside, 0]).abs().max()) < 0.05 * float(v[inside, 0].abs().max()) + 0.05
        table = order[at:at + -(-n // P)]
        at += len(table)
        first_needed = max(0, n - ql - window + 1) // P       # pages in front of every window: gone
        for i, pg in enumerate(table):
            bt[r, i] = pg if i >= first_needed else -1
        for i in range(n):
            k_pool[table[i // P], :, i % P] = k[i]
            v_pool[table[i // P], :, i % P] = v[i]
        qs.append(q), want.append(out)
    want_all = torch.cat(want)
    q_all = dev(torch.cat(qs), dtype)
    kp, vp = dev(k_pool, dtype), dev(v_pool, dtype)
    q_start, ctx = i32([0, qlens[0], qlens[0] + 1]), i32(lens)
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    ws, wo = work_items(qlens, lens, 0, 16)
    out = torch.empty(q_all.shape[0], H, Dv, dtype=dtype, device="cuda")
    ops.attention_generic_kv(out, q_all, kp, vp, q_start, ctx, bt.cuda(), torch.from_numpy(ws).cuda(),
                             torch.from_numpy(wo).cuda(), scale, 1, window)
    assert float((out.double().cpu() - want_all).abs().max()) < tol * float(want_all.abs().max())
    if ops.attention_decode_kv_fits(Dk, Dv):
        # the decoded token alone, as the leading sequence of a step, over 1 and 3 workgroups
        for splits in (1, 3):
            out = torch.empty(1, H, Dv, dtype=dtype, device="cuda")
            ops.attention_decode_kv(out, dev(qs[1], dtype), kp, vp, i32([0, 1]), i32(lens[1:]), bt[1:].cuda(), 1,
                                    scale, 1, splits, window)
            assert float((out.double().cpu() - want[1]).abs().max()) < tol * float(want[1].abs().max())
    if ops.attention_prefill_mfma_kv_fits(dtype, G, 1, Dk, Dv, P):
        ws, wo = work_items(qlens, lens, 0, 64)
        out = torch.empty(q_all.shape[0], H, Dv, dtype=dtype, device="cuda")
        ops.attention_prefill_mfma_kv(out, q_all, kp, vp, q_start, ctx, bt.cuda(), torch.from_numpy(ws).cuda(),
                                      torch.from_numpy(wo).cuda(), scale, 1, len(ws), window)
        assert float((out.double().cpu() - want_all).abs().max()) < 1.5e-2 * float(want_all.abs().max())
