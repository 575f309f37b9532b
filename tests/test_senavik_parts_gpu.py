"""The mechanisms that the Senavik design added, each alone, against the plain functions of
tests/plain_senavik.py or a few lines of float64 arithmetic: the kept first tokens, the window's
edges and the denominator's extra term in every attention kernel (prompt portions and decoding,
shuffled pages, pages given back), the choice of experts by groups, the latent mixer's rotation in
the half layout with queries from a matrix of their own, the norm behind the embedding, the norm
of a range of columns, and the two mixers and the routed feed-forward as parts."""
import math

import pytest
import torch

import plain_senavik as ps

pytestmark = pytest.mark.gpu


def dev(t, dtype=torch.float32):
    return t.to("cuda", dtype).contiguous()


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# ---- windows, kept tokens and sinks in the attention kernels ----------------------------------------
def _attend(q, k, v, n, ql, window, keep, scale, H, G, sink):
    """The last ql of n positions: softmax over the visible keys with the sink in the denominator."""
    vis = ps.visible(n, window, keep)[n - ql:] if window else ps.visible(n)[n - ql:]
    out = torch.zeros(ql, H, v.shape[-1], dtype=torch.float64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        out[:, h] = ps.sink_softmax(s, vis, sink[h] if sink is not None else None) @ v[:, g]
    return out


CASES = [  # H, G, Dk, Dv, window, keep, page
    (4, 2, 32, 64, 33, 17, 16),      # matrix-core prompt kernel, split-KV vector kernel; kept: more than a page
    (4, 2, 64, 64, 40, 16, 16),      # both matrix-core kernels; kept: exactly a page
    (8, 2, 128, 128, 64, 4, 16),     # four heads a kv head, the largest matrix-core size
    (2, 1, 16, 48, 24, 8, 8),        # vector kernels
    (3, 3, 20, 12, 7, 3, 4),         # sizes the split-KV kernel does not take
    (2, 2, 32, 32, 1, 2, 8),         # a window of one: the query itself and the kept tokens
    (4, 4, 64, 64, 20, 30, 16),      # more kept tokens than the window is long
    (2, 1, 96, 96, 50, 0, 16),       # a window that keeps nothing
    (4, 1, 64, 64, 0, 0, 16),        # no window: the sink alone
    (5, 5, 80, 80, 0, 0, 4),         # one "kv head" a query head with a size the matrix cores do not take
]


@pytest.mark.parametrize("sinks", [True, False], ids=["sink", "nosink"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("H,G,Dk,Dv,window,keep,P", CASES)
def test_kept_tokens_window_edges_and_sinks_in_every_kernel(gpu_device, dtype, sinks, H, G, Dk, Dv, window, keep, P):
    """A portion of a prompt behind a cached prefix, a long portion from the start, and a single
    decoded token, through every kernel that takes the sizes. For the last query of each sequence
    one head's query points at the last kept key (position keep - 1), which must get its weight,
    and the key behind it (position keep) is made so that it would win if it were seen. Pages
    between the kept ones and the windows are not there (table entries -1)."""
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.engine.batch import work_items
    torch.manual_seed(window * 7 + keep + Dk)
    pages, scale = 176, 0.3
    lens, qlens = [150, 300, 205], [40, 300, 1]
    order = torch.randperm(pages).tolist()
    k_pool = torch.randn(pages, G, P, Dk, dtype=torch.float64) * 5
    v_pool = torch.randn(pages, G, P, Dv, dtype=torch.float64) * 5
    bt = torch.full((3, -(-max(lens) // P)), -1, dtype=torch.int32)
    sink = torch.randn(H, dtype=torch.float64) * 2 if sinks else None
    if sinks:
        sink[-1] = 9.0                       # one head whose sink outweighs its keys
    qs, want, at = [], [], 0
    for r, (n, ql) in enumerate(zip(lens, qlens)):
        k = torch.randn(n, G, Dk, dtype=torch.float64)
        v = torch.randn(n, G, Dv, dtype=torch.float64)
        q = torch.randn(ql, H, Dk, dtype=torch.float64)
        if window and keep:
            k[keep - 1] *= 3.0
            q[-1, 0] = k[keep - 1, 0] * (32.0 / Dk)
            if keep < n - window:
                k[keep] = k[keep - 1] * 1.5          # would win if it were seen
        if window and n - window >= 0:
            k[n - window] *= 2.0                      # the window's first key, and the one in front of it
            q[-1, 1] = k[n - window, 1 // (H // G)] * (32.0 / Dk)
            if n - window - 1 >= keep:
                k[n - window - 1] = k[n - window] * 1.5
        if dtype == torch.bfloat16:
            q, k, v = (t.bfloat16().double() for t in (q, k, v))
        out = _attend(q, k, v, n, ql, window, keep, scale, H, G, sink)
        table = order[at:at + -(-n // P)]
        at += len(table)
        first_needed = max(0, n - ql - window + 1) // P if window else 0
        kept_pages = -(-keep // P)
        for i, pg in enumerate(table):
            bt[r, i] = pg if (i >= first_needed or i < kept_pages) else -1
        for i in range(n):
            k_pool[table[i // P], :, i % P] = k[i]
            v_pool[table[i // P], :, i % P] = v[i]
        qs.append(q), want.append(out)
    want_all = torch.cat(want)
    q_all = dev(torch.cat(qs), dtype)
    kp, vp = dev(k_pool, dtype), dev(v_pool, dtype)
    sk = dev(sink) if sinks else None
    q_start, ctx = i32([0, 40, 340, 341]), i32(lens)
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    top = float(want_all.abs().max())
    extras = dict(keep_first=keep, sink=sk)
    ws, wo = work_items(qlens, lens, 0, 16)
    out = torch.empty(q_all.shape[0], H, Dv, dtype=dtype, device="cuda")
    ops.attention_generic_kv(out, q_all, kp, vp, q_start, ctx, bt.cuda(), torch.from_numpy(ws).cuda(),
                             torch.from_numpy(wo).cuda(), scale, 1, window, **extras)
    assert float((out.double().cpu() - want_all).abs().max()) < tol * top
    same = Dk == Dv
    if same:        # the entry points for keys and values of one size (what the latent mixer calls)
        out = torch.empty(q_all.shape[0], H, Dv, dtype=dtype, device="cuda")
        ops.attention_generic(out, q_all, kp, vp, q_start, ctx, bt.cuda(), torch.from_numpy(ws).cuda(),
                              torch.from_numpy(wo).cuda(), scale, window, **extras)
        assert float((out.double().cpu() - want_all).abs().max()) < tol * top
    q_dec, bt_dec = dev(qs[2], dtype), bt[2:].cuda()
    if ops.attention_decode_kv_fits(Dk, Dv):
        for splits in (1, 3):
            out = torch.empty(1, H, Dv, dtype=dtype, device="cuda")
            ops.attention_decode_kv(out, q_dec, kp, vp, i32([0, 1]), i32(lens[2:]), bt_dec, 1, scale, 1, splits,
                                    window, **extras)
            assert float((out.double().cpu() - want[2]).abs().max()) < tol * top, splits
    if same and ops.attention_decode_mfma_fits(dtype, H, G, Dk, P):
        for splits in (1, 2, 5):
            out = torch.empty(1, H, Dv, dtype=dtype, device="cuda")
            ops.attention_decode(out, q_dec, kp, vp, i32([0, 1]), i32(lens[2:]), bt_dec, 1, scale, window, splits,
                                 matrix_cores=True, **extras)
            assert float((out.double().cpu() - want[2]).abs().max()) < 1.5e-2 * top, splits
    if ops.attention_prefill_mfma_kv_fits(dtype, G, 1, Dk, Dv, P):
        ws, wo = work_items(qlens, lens, 0, 64)
        for groups in (len(ws), 2):
            out = torch.empty(q_all.shape[0], H, Dv, dtype=dtype, device="cuda")
            ops.attention_prefill_mfma_kv(out, q_all, kp, vp, q_start, ctx, bt.cuda(), torch.from_numpy(ws).cuda(),
                                          torch.from_numpy(wo).cuda(), scale, 1, groups, window, **extras)
            assert float((out.double().cpu() - want_all).abs().max()) < 1.5e-2 * top, groups
    if same and ops.attention_prefill_mfma_fits(dtype, G, Dk, P):
        for rows in (64, 128):
            ws, wo = work_items(qlens, lens, 0, rows)
            out = torch.empty(q_all.shape[0], H, Dv, dtype=dtype, device="cuda")
            ops.attention_prefill_mfma(out, q_all, kp, vp, q_start, ctx, bt.cuda(), torch.from_numpy(ws).cuda(),
                                       torch.from_numpy(wo).cuda(), scale, window, rows, 0, **extras)
            assert float((out.double().cpu() - want_all).abs().max()) < 1.5e-2 * top, rows


def test_a_sink_needs_a_head_each_and_kept_tokens_a_window(gpu_device):
    from pytriton_llama_amd import ops
    q = torch.zeros(1, 2, 16, device="cuda")
    pool = torch.zeros(2, 1, 4, 16, device="cuda")
    args = (torch.empty_like(q), q, pool, pool, i32([0, 1]), i32([1]), i32([[0]]), 1, 0.5, 1, 1)
    with pytest.raises(ops.KernelError):
        ops.attention_decode_kv(*args, 0, keep_first=0, sink=torch.zeros(3, device="cuda"))
    with pytest.raises(ops.KernelError):
        ops.attention_decode_kv(*args, 0, keep_first=2, sink=None)
    ops.attention_decode_kv(*args, 4, keep_first=2, sink=torch.zeros(2, device="cuda"))


# ---- the choice of experts by groups ---------------------------------------------------------------
@pytest.mark.parametrize("E,count,keep,top", [(8, 4, 2, 2), (6, 3, 2, 3), (16, 4, 3, 2), (4, 4, 3, 2), (12, 1, 1, 4),
                                              (64, 8, 4, 8), (130, 10, 3, 6), (9, 3, 3, 5), (6, 6, 2, 2), (256, 64, 5, 7)])
def test_router_with_groups(gpu_device, E, count, keep, top):
    """Sigmoid scores, a correction for the choice alone, groups scored by their two best choice
    scores (groups of one: by their only one), weights from the plain scores of the chosen,
    divided by their sum. The corrections are large and partly negative, so that choice scores
    below zero occur and the groups that win are not those of the largest plain scores."""
    from pytriton_llama_amd import ops
    torch.manual_seed(E + count)
    T = 61
    z = torch.randn(T, E, dtype=torch.float64) * 2
    corr = torch.randn(E, dtype=torch.float64) * 0.7 - 0.5
    mlp = {"router": {"experts": E, "top": top, "groups": {"count": count, "keep": keep}}}
    w = {"router": torch.eye(E, dtype=torch.float64), "correction": corr.float().double()}
    zz = z.float().double()
    ps.ROUTER_MARGINS, margin = [], ps.CLOSE_CALL
    ps.CLOSE_CALL = 1e-5                    # (float32 against float64: only near-ties can differ)
    try:
        idx, wgt = ps.route(zz, mlp, w)
        close = ps.ROUTER_MARGINS[0]
    finally:
        ps.ROUTER_MARGINS, ps.CLOSE_CALL = None, margin
    r = ops.moe_route(dev(z), E, top, 0, True, ops.SCORE_SIGMOID, dev(corr), 0, 1e-20, 1.0, count, keep)
    mine, mw = r.idx.view(T, top).cpu().long(), r.wgt.view(T, top).cpu().double()
    sure = ~close                           # float32 sums may turn a choice the float64 margin calls close
    assert int(sure.sum()) > T - 4
    a, b = mine.sort(-1), idx.sort(-1)
    assert torch.equal(a.values[sure], b.values[sure])
    assert float((mw.gather(1, a.indices) - wgt.gather(1, b.indices))[sure].abs().max()) < 1e-5
    assert float((mw.sum(-1) - 1.0).abs().max()) < 1e-5
    # what the groups are for: without them other experts are chosen somewhere
    free, _ = ps.route(zz, {"router": {"experts": E, "top": top}}, w)
    if keep < count and E >= 16:
        assert not torch.equal(free.sort(-1).values, idx.sort(-1).values)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("E,count,keep,top,I", [(8, 4, 2, 2, 40), (6, 3, 3, 3, 24), (5, 1, 1, 1, 33)])
def test_routed_feed_forward_as_a_part(gpu_device, dtype, E, count, keep, top, I):
    from pytriton_llama_amd.parts import build_part
    torch.manual_seed(E + I)
    W, T = 48, 37
    part = build_part("feed_forward", "routed_experts", hidden_size=W, intermediate_size=I, num_experts=E, top=top,
                      activation="silu", weight_on_input=False, renormalize=True, renorm_eps=1e-20, score="sigmoid",
                      correction_name="correction", groups=(count, keep), shared=None, shared_gate=False)
    w = {}
    for src in part.param_sources():
        w[src.name] = {"correction": 0.5, "router": 0.4}.get(src.name, 0.2) * torch.randn(src.shape)
        if src.kind == "matrix" and dtype == torch.bfloat16:
            w[src.name] = w[src.name].bfloat16().float()
    part.load(w, dtype, "cuda")
    h = torch.randn(T, W)
    if dtype == torch.bfloat16:
        h = h.bfloat16().float()
    got = part.forward(dev(h, dtype)).double().cpu()
    mlp = {"router": {"experts": E, "top": top, "groups": {"count": count, "keep": keep}}}
    ps.ROUTER_MARGINS = []
    try:
        want = ps.routed_ff(h.double(), mlp, {k: v.double() for k, v in w.items()})
        close = ps.ROUTER_MARGINS[0]
    finally:
        ps.ROUTER_MARGINS = None
    err = ((got - want).abs().amax(-1) / want.abs().max())[~close]
    assert float(err.max()) < (2e-5 if dtype == torch.float32 else 2e-2)


def test_dense_feed_forward_as_a_part(gpu_device):
    from pytriton_llama_amd.parts import build_part
    torch.manual_seed(3)
    part = build_part("feed_forward", "mlp", hidden_size=40, intermediate_size=56, activation="relu2")
    w = {s.name: 0.3 * torch.randn(s.shape) for s in part.param_sources()}
    part.load(w, torch.float32, "cuda")
    h = torch.randn(19, 40)
    want = ps.dense_ff(h.double(), {k: v.double() for k, v in w.items()})
    assert float((part.forward(dev(h)).double().cpu() - want).abs().max()) < 2e-5 * float(want.abs().max())


# ---- the latent mixer's preparation ----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("H,dn,dr,R,dims,half", [(3, 8, 12, 20, 12, True), (2, 10, 6, 18, 4, True), (4, 16, 16, 48, 16, True),
                                                 (1, 0, 8, 32, 8, True), (2, 6, 8, 24, 6, False)])
def test_latent_preparation_in_the_half_layout(gpu_device, dtype, H, dn, dr, R, dims, half):
    """Queries from a matrix of their own, the down-projection from another; entry i of the
    rotating entries turns with entry i + dims / 2 (or with its neighbour), sine and cosine times a
    factor; positions beyond a thousand; the latent normed in float32; a padding row writes nothing."""
    from pytriton_llama_amd import ops
    torch.manual_seed(H + dr)
    T, P, pages, eps, mag = 9, 4, 6, 1e-5, 1.1386
    D = R + dr
    pos = torch.tensor([0, 1, 2, 3, 1000, 1001, 4097, 5, 6])
    queries = torch.randn(T, 5 + H * (dn + dr))
    proj = torch.randn(T, 7 + D + 3)
    cw = 1 + 0.1 * torch.randn(R)
    if dtype == torch.bfloat16:
        queries, proj = queries.bfloat16().float(), proj.bfloat16().float()
    freqs, _ = ps.ramped_freqs(5000.0, dims, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0})
    f32 = freqs.float()
    slots = torch.tensor([3, 2, 1, 0, 7, 6, 5, -1, 9], dtype=torch.int32)
    pool = torch.zeros(pages, 1, P, D, dtype=dtype, device="cuda")
    q_out = torch.zeros(T, H, D, dtype=dtype, device="cuda")
    ops.latent_prepare(q_out, dev(proj, dtype), 5, 7, pos.int().cuda(), dev(f32), dev(cw), eps, slots.cuda(), pool,
                       H, dn, dr, R, queries=dev(queries, dtype), half_layout=half, mag=mag)

    def turn(x):           # x [T, heads, dr]
        if half:
            return ps.rotate_half(x, pos, dims, f32.double(), mag)
        a = pos.double()[:, None] * f32.double()[None, :]
        c, s = (torch.cos(a) * mag)[:, None, :], (torch.sin(a) * mag)[:, None, :]
        y = x.clone()
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        y[..., 0:dims:2], y[..., 1:dims:2] = u * c - v * s, v * c + u * s
        return y
    qr = queries.double()[:, 5:5 + H * (dn + dr)].view(T, H, dn + dr)[:, :, dn:]
    tol = 3e-4 if dtype == torch.float32 else 2e-2          # (float32 angles at position 4097)
    assert float((q_out.double().cpu()[:, :, R:] - turn(qr)).abs().max()) < tol * 4
    assert float(q_out.double().cpu()[:, :, :R].abs().max()) == 0.0
    down = proj.double()[:, 7:7 + D]
    c = ps.rms(down[:, :R], eps) * cw.double()
    kr = turn(down[:, None, R:])[:, 0]
    flat = pool.double().cpu().view(pages * P, D)
    for t in range(T):
        if slots[t] < 0:
            continue
        assert float((flat[slots[t], :R] - c[t]).abs().max()) < tol * 4
        assert float((flat[slots[t], R:] - kr[t]).abs().max()) < tol * 4
    assert float(flat[8].abs().max()) == 0.0 and float(flat[4].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["latent", "attention"])
def test_mixers_as_parts_over_a_fresh_cache(gpu_device, dtype, name):
    """One mixer alone, a whole prompt, against the plain function."""
    from pytriton_llama_amd.cache import CacheManager, CacheStorage
    from pytriton_llama_amd.engine.batch import StepEntry, build_context
    from pytriton_llama_amd.parts import build_part
    torch.manual_seed(11)
    W, T, eps = 40, 53, 1e-5
    if name == "latent":
        m = {"heads": 3, "dim": 8, "rot_dim": 12, "vdim": 12, "kv_rank": 20, "q_rank": 16, "scale": 0.25,
             "rot": {"base": 5000.0, "dims": 12, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}}
        part = build_part("mixer", "latent_attention", hidden_size=W, num_heads=3, dim=8, rot_dim=12, vdim=12, kv_rank=20,
                          scale=0.25, rot_base=5000.0, rot_dims=12, eps=eps, gated=False, q_rank=16, rot_layout="half",
                          rot_scaling=m["rot"]["scaling"], sink_name="sink")
    else:
        m = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "mask": {"size": 20, "keep_first": 3},
             "rot": {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}}
        part = build_part("mixer", "normed_attention", hidden_size=W, num_heads=4, num_kv_heads=2, dim=16, vdim=24,
                          scale=0.3, eps=eps, qk_norm=None, maps=1, bias=False, gated=False, rot_dims=8, rot_base=10000.0,
                          rot_scaling=m["rot"]["scaling"], window=20, keep_first=3, sink_name="sink")
    w = {}
    for src in part.param_sources():
        w[src.name] = (1 + 0.1 * torch.randn(src.shape)) if src.name.endswith("norm") else 0.3 * torch.randn(src.shape)
        if src.kind == "matrix" and dtype == torch.bfloat16:
            w[src.name] = w[src.name].bfloat16().float()
    part.load(w, dtype, "cuda")
    h = torch.randn(T, W)
    if dtype == torch.bfloat16:
        h = h.bfloat16().float()
    man = CacheManager([part.cache_spec()], 4, 32, 2)
    store = CacheStorage(man, dtype, torch.device("cuda:0"))
    man.admit("a")
    ctx, _ = build_context([StepEntry("a", list(range(T)), ())], man, torch.device("cuda:0"), None, part.work_lists())
    y = part.forward(dev(h, dtype), ctx, store.view(0, True))
    y = y.tensor() if hasattr(y, "tensor") else y
    w64 = {k: v.double() for k, v in w.items()}
    want = ps.latent_attention(h.double(), m, w64, eps, torch.arange(T)) if name == "latent" else \
        ps.attention(h.double(), m, w64, torch.arange(T))
    assert float((y.double().cpu() - want).abs().max()) < (2e-5 if dtype == torch.float32 else 3e-2) * float(want.abs().max())


# ---- norms -----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("H", [24, 64, 257, 1024, 3000])
def test_norm_behind_the_embedding_and_norm_of_columns(gpu_device, dtype, H):
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.parts import build_part
    torch.manual_seed(H)
    V, T, eps = 50, 13, 1e-5
    table = torch.randn(V, H)
    if dtype == torch.bfloat16:
        table = table.bfloat16().float()
    w = 0.2 * torch.randn(H)
    ids = torch.randint(0, V, (T,))
    norm = build_part("norm", "rmsnorm", size=H, eps=eps, weight_name="", offset=1.0)
    emb = build_part("embedding", "token_embedding", vocab_size=V, hidden_size=H, weight_name="embed", float32_stream=True,
                     norm=norm)
    assert [s.name for s in emb.param_sources()] == ["embed", "embed.norm"]
    emb.load({"embed": table, "embed.norm": w}, dtype, "cuda")
    got = emb.forward(ids.int().cuda())
    want = ps.offset_norm(table.double()[ids], w.double(), eps)
    assert got.dtype == torch.float32 and float((got.double().cpu() - want).abs().max()) < 1e-5 * float(want.abs().max())
    # the same norm on rows of a float32 stream, for the engine's dtype
    y, _ = norm.forward(got, None)
    assert y.dtype == dtype
    again = ps.offset_norm(want, w.double(), eps)
    assert float((y.double().cpu() - again).abs().max()) < (1e-5 if dtype == torch.float32 else 1e-2) * float(again.abs().max())
    # a range of columns of a wider matrix, with a plain weight
    wide = torch.randn(T, H + 21)
    if dtype == torch.bfloat16:
        wide = wide.bfloat16().float()
    pw = 1 + 0.1 * torch.randn(H)
    cols = ops.rmsnorm_cols(dev(wide, dtype)[:, 8:8 + H], dev(pw), eps)
    want = ps.rms(wide.double()[:, 8:8 + H], eps) * pw.double()
    assert cols.is_contiguous() and float((cols.double().cpu() - want).abs().max()) < (1e-5 if dtype == torch.float32 else 1e-2) * float(want.abs().max())
