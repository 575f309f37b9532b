"""Senavik's configuration and builder on the CPU, the cache manager's kept first pages, the
frequency rules of the package against the plain ones, and the plain implementation's mechanisms
against special cases worked out by hand."""
import math

import pytest
import torch

import plain_senavik as ps
from senavik_configs import SENAVIK, senavik


def test_config_reads_every_size_and_constant():
    from pytriton_llama_amd.config import SenavikConfig
    cfg, _, _ = senavik("S1")
    c = SenavikConfig.from_dict(cfg)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, len(c.layers)) == (200, 64, 1e-5, 4)
    assert [l.kind for l in c.layers] == ["attention", "latent_attention", "attention", "latent_attention"]
    a, l = c.layers[0].mixer, c.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.window, a.keep_first, a.rot_dims, a.rot_base) == \
        (4, 2, 16, 24, 0.3, 20, 3, 8, 10000.0)
    assert a.rot_scaling == {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64.0}
    assert (l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank, l.q_rank, l.scale, l.rot_dims, l.rot_base) == \
        (3, 8, 12, 12, 20, 16, 0.25, 12, 5000.0)
    assert l.rot_scaling == {"factor": 4.0, "original": 32.0, "fast": 8.0, "slow": 1.0}
    m, d = c.layers[0].mlp, c.layers[1].mlp
    assert (m.kind, m.ff, m.experts, m.top, m.groups, m.keep_groups) == ("moe", 40, 8, 2, 4, 2)
    assert (d.kind, d.ff) == ("dense", 48) and c.layers[2].mlp is None
    assert c.to_dict() == cfg
    other = SenavikConfig.from_dict(senavik("S2")[0])
    b = other.layers[1].mixer
    assert (b.window, b.keep_first, b.rot_dims, b.rot_scaling) == (None, 0, 0, None)
    assert other.layers[2].mixer.keep_first == 0 and other.layers[0].mlp.groups == 1
    assert other.layers[0].mixer.rot_dims == 4 and other.layers[3].mixer.rot_scaling is None


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][0].update(type="mamba1"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "lacks 'scale'"),
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "dims 18"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size must be positive"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(keep_first=-1), "keep_first"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("high"), "lacks 'high'"),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "lacks 'q_rank'"),
    (lambda c: c["layers"][1]["mixer"].update(rot_dim=7), "dims 12"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("slow"), "lacks 'slow'"),
    (lambda c: c["layers"][1]["mixer"].update(kv_rank=640), "up to 640"),
    (lambda c: c["layers"][0]["mlp"].update(kind="shared"), "unknown feed-forward kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top 9 of 8"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=5), "groups"),
    (lambda c: c["layers"][3]["mlp"]["router"]["groups"].update(keep=1), "groups"),
    (lambda c: c["layers"][1]["mlp"].pop("ff"), "lacks 'ff'"),
    (lambda c: c.pop("norm"), "lacks 'norm'"),
    (lambda c: c.update(layers=[]), "empty"),
])
def test_config_errors_name_the_place(change, text):
    from pytriton_llama_amd.config import ConfigError, SenavikConfig
    cfg, _, _ = senavik("S1")
    change(cfg)
    with pytest.raises(ConfigError) as e:
        SenavikConfig.from_dict(cfg)
    assert text in str(e.value)


@pytest.mark.parametrize("name", sorted(SENAVIK))
def test_builder_wires_caches_and_names(name):
    import pytriton_llama_amd  # noqa: F401
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.parts import PagedSpec
    cfg, _, _ = senavik(name)
    model = build_model(cfg)
    assert [c.block for c in model.schedule] == list(range(len(cfg["layers"])))
    assert [c.cache_layer for c in model.schedule] == list(range(len(cfg["layers"])))
    names = model.expected_tensors()
    assert {"embed", "embed.norm", "final.norm", "head", "l0.norm1"} <= set(names)
    assert names["head"][1].shape == (cfg["vocab"], cfg["width"])
    for i, layer in enumerate(cfg["layers"]):
        m, spec = layer["mixer"], model.cache_layers[i]
        assert isinstance(spec, PagedSpec)
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None)
        assert names[f"l{i}.mix.sink"][1].shape == (m["heads"],)
        if layer["type"] == "attention":
            mask = m.get("mask") or {}
            assert (spec.window, spec.keep_first) == (mask.get("size"), mask.get("keep_first", 0))
            assert [t.name for t in spec.tensors] == ["k", "v"]
            assert spec.tensors[0].shape == (m["kv_heads"], m["dim"]) and spec.tensors[1].shape == (m["kv_heads"], m["vdim"])
            assert {f"l{i}.mix.q", f"l{i}.mix.k", f"l{i}.mix.v", f"l{i}.mix.o"} <= set(names)
            assert f"l{i}.mix.q.norm" not in names and f"l{i}.mix.q.b" not in names
        else:
            assert spec.window is None and [t.name for t in spec.tensors] == ["latent"]
            assert spec.tensors[0].shape == (1, m["kv_rank"] + m["rot_dim"])
            assert names[f"l{i}.mix.dq"][1].shape == (m["q_rank"], cfg["width"])
            assert names[f"l{i}.mix.dq.norm"][1].shape == (m["q_rank"],)
            assert names[f"l{i}.mix.uq"][1].shape == (m["heads"] * (m["dim"] + m["rot_dim"]), m["q_rank"])
            assert names[f"l{i}.mix.dkv"][1].shape == (m["kv_rank"] + m["rot_dim"], cfg["width"])
            assert names[f"l{i}.mix.dkv.norm"][1].shape == (m["kv_rank"],)
            assert names[f"l{i}.mix.uk"][1].shape == (m["heads"] * m["dim"], m["kv_rank"])
            assert names[f"l{i}.mix.uv"][1].shape == (m["heads"] * m["vdim"], m["kv_rank"])
            assert f"l{i}.mix.q" not in names and f"l{i}.mix.g" not in names
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "moe":
            E = mlp["router"]["experts"]
            assert names[f"l{i}.mlp.router"][1].shape == (E, cfg["width"])
            assert names[f"l{i}.mlp.correction"][1].shape == (E,)
            assert f"l{i}.mlp.e{E - 1}.gate" in names and f"l{i}.mlp.e{E}.up" not in names
        elif mlp is not None:
            assert names[f"l{i}.mlp.up"][1].shape == (mlp["ff"], cfg["width"]) and f"l{i}.mlp.gate" not in names


def test_kept_first_pages_are_never_given_back():
    """A window of 6 over pages of 4 that keeps 9 tokens: the three pages of positions 0..11 stay,
    the pages between them and the window go back, and a group without kept tokens gives all back."""
    from pytriton_llama_amd.cache import RELEASED, CacheManager
    from pytriton_llama_amd.parts import PagedSpec, PagedTensor
    kv = (PagedTensor("k", (1, 8), 1), PagedTensor("v", (1, 8), 1))
    man = CacheManager([PagedSpec(kv, 6, 9), PagedSpec(kv, 6, 0), PagedSpec(kv, None, 0)], 4, 40, 2)
    assert len(man.paged) == 3
    man.admit("a")
    man.append("a", 50)
    assert man.release_behind_window("a") == (11 - 3) + 11
    kept, plain, full = (man.block_table("a", g) for g in range(3))
    assert all(p >= 0 for p in kept[:3]) and all(p == RELEASED for p in kept[3:11]) and all(p >= 0 for p in kept[11:])
    assert all(p == RELEASED for p in plain[:11]) and all(p >= 0 for p in full)
    man.check()
    man.append("a", 30)
    man.release_behind_window("a")
    assert [i for i, p in enumerate(man.block_table("a", 0)) if p >= 0] == [0, 1, 2, 18, 19]
    man.free("a")
    man.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in man.paged)
    # kept tokens that the window still covers: nothing between them and the window to give back
    man.admit("b")
    man.append("b", 13)
    assert man.release_behind_window("b") == 2          # (both from the group that keeps nothing)
    assert all(p >= 0 for p in man.block_table("b", 0))


# ---- the package's frequency rules against the plain ones -----------------------------------------
@pytest.mark.parametrize("base,dims,scaling", [
    (10000.0, 8, (4.0, 1.0, 4.0, 64)), (500000.0, 64, (8.0, 1.0, 4.0, 8192)), (800.0, 8, (4.0, 1.0, 2.0, 40)),
    (100.0, 6, (2.0, 2.0, 3.0, 40)), (10000.0, 32, (16.0, 0.5, 8.0, 100))])
def test_banded_frequencies(base, dims, scaling):
    from pytriton_llama_amd.parts import banded_inv_freq
    want, mag = ps.banded_freqs(base, dims, dict(zip(("factor", "low", "high", "original"), scaling)))
    got = banded_inv_freq(base, dims, *scaling[:3], scaling[3])
    assert mag == 1.0 and got.dtype == torch.float32
    assert torch.allclose(got.double(), want, rtol=1e-7, atol=0)
    plain = ps.plain_freqs(base, dims)
    kept, slowed = torch.isclose(want, plain), torch.isclose(want, plain / scaling[0])
    assert kept[0] and slowed[-1]          # the fastest entry stays, the slowest is divided
    if (base, dims) in ((10000.0, 8), (500000.0, 64)):
        assert not (kept | slowed).all()   # and some entry lies between the bands


@pytest.mark.parametrize("base,dims,scaling", [
    (5000.0, 12, (4.0, 32, 8.0, 1.0)), (800.0, 4, (8.0, 32, 64.0, 16.0)), (20000.0, 16, (2.0, 64, 16.0, 2.0)),
    (10000.0, 64, (40.0, 4096, 32.0, 1.0)), (10000.0, 8, (4.0, 16, 4.0, 1.0))])
def test_ramped_frequencies(base, dims, scaling):
    from pytriton_llama_amd.parts import ramp_inv_freq
    want, mag = ps.ramped_freqs(base, dims, dict(zip(("factor", "original", "fast", "slow"), scaling)))
    got, got_mag = ramp_inv_freq(base, dims, *scaling)
    assert torch.allclose(got.double(), want, rtol=1e-7, atol=0)
    assert abs(got_mag - mag) < 1e-12 and abs(mag - (0.1 * math.log(scaling[0]) + 1.0)) < 1e-12
    plain = ps.plain_freqs(base, dims)
    assert torch.isclose(want[-1], plain[-1] / scaling[0])      # the slowest entry is divided


def test_ramp_whose_ends_coincide():
    """fast and slow so large that both ends fall before the first entry: the ramp is a step from
    the first entry (unscaled) to the second (divided)."""
    want, _ = ps.ramped_freqs(800.0, 4, {"factor": 8.0, "original": 32, "fast": 64.0, "slow": 16.0})
    plain = ps.plain_freqs(800.0, 4)
    assert torch.allclose(want, torch.stack([plain[0], plain[1] / 8.0]))


# ---- the plain implementation against special cases --------------------------------------------
def test_plain_window_with_kept_tokens():
    vis = ps.visible(8, 3, 2)
    assert vis[7].tolist() == [True, True, False, False, False, True, True, True]
    assert vis[3].tolist() == [True, True, True, True, False, False, False, False]
    assert vis[4].tolist() == [True, True, True, True, True, False, False, False]
    assert ps.visible(8, 3, 0)[7].tolist() == [False] * 5 + [True] * 3
    assert ps.visible(5).sum() == 15 and ps.visible(5, 1, 0).sum() == 5
    assert ps.visible(6, 1, 2)[5].tolist() == [True, True, False, False, False, True]


def test_plain_softmax_with_a_sink():
    s = torch.tensor([[0.0, 0.0], [math.log(3.0), 0.0]], dtype=torch.float64)
    vis = torch.tensor([[True, False], [True, True]])
    p = ps.sink_softmax(s, vis, torch.tensor(0.0, dtype=torch.float64))
    assert torch.allclose(p, torch.tensor([[0.5, 0.0], [0.6, 0.2]], dtype=torch.float64))
    # a sink far below the scores changes nothing, one far above takes everything
    assert torch.allclose(ps.sink_softmax(s, vis, torch.tensor(-800.0, dtype=torch.float64)), ps.sink_softmax(s, vis, None))
    assert float(ps.sink_softmax(s, vis, torch.tensor(800.0, dtype=torch.float64)).sum()) < 1e-300


def test_plain_rotation_is_a_rotation():
    x = torch.randn(5, 2, 8, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 1000])
    f = ps.plain_freqs(100.0, 4)
    y = ps.rotate_half(x, pos, 4, f)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    assert torch.allclose(y[..., :4].norm(dim=-1), x[..., :4].norm(dim=-1))
    assert torch.allclose(ps.rotate_half(x, pos, 4, f, 1.5)[..., :4], 1.5 * y[..., :4])
    # entry 0 turns with entry 2, entry 1 with entry 3
    e = torch.zeros(1, 1, 4, dtype=torch.float64)
    e[0, 0, 0] = 1.0
    r = ps.rotate_half(e, torch.tensor([1]), 4, f)[0, 0]
    assert torch.allclose(r, torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0], dtype=torch.float64))
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    f8 = ps.plain_freqs(50.0, 8)
    a = (ps.rotate_half(q, torch.tensor([7]), 8, f8) * ps.rotate_half(k, torch.tensor([3]), 8, f8)).sum()
    b = (ps.rotate_half(q, torch.tensor([104]), 8, f8) * ps.rotate_half(k, torch.tensor([100]), 8, f8)).sum()
    assert abs(float(a - b)) < 1e-9


def test_plain_router_groups():
    """Eight experts in four pairs, two pairs kept, two experts chosen. Token 0: the largest single
    score sits in a pair whose sum loses, so it is not chosen. The correction moves the choice
    and not the weights."""
    mlp = {"router": {"experts": 8, "top": 2, "groups": {"count": 4, "keep": 2}}}
    z = torch.tensor([[3.0, -9.0, 1.0, 1.2, 0.8, 1.1, -9.0, -9.0]], dtype=torch.float64)
    w = {"router": z.T.contiguous() @ torch.ones(1, 1, dtype=torch.float64), "correction": torch.zeros(8, dtype=torch.float64)}
    h = torch.ones(1, 1, dtype=torch.float64)
    s = torch.sigmoid(z[0])
    # pair sums: (s0 + s1, s2 + s3, s4 + s5, s6 + s7) -> pairs 1 and 2 win over pair 0
    assert float(s[2] + s[3]) > float(s[0] + s[1]) and float(s[4] + s[5]) > float(s[0] + s[1])
    idx, wgt = ps.route(h, mlp, w)
    assert idx[0].tolist() == [3, 5]
    assert torch.allclose(wgt[0], torch.stack([s[3], s[5]]) / (s[3] + s[5]))
    # without groups the largest score wins
    idx, _ = ps.route(h, {"router": {"experts": 8, "top": 2}}, w)
    assert idx[0].tolist() == [0, 3]
    # a correction that lifts pair 3 above all: its experts are chosen, with their own small scores
    w["correction"] = torch.tensor([0, 0, 0, 0, 0, 0, 5.0, 5.0], dtype=torch.float64)
    idx, wgt = ps.route(h, mlp, w)
    assert sorted(idx[0].tolist()) == [6, 7] and torch.allclose(wgt[0], torch.full((2,), 0.5, dtype=torch.float64))
    # negative choice scores: an expert outside the kept groups is not chosen even if its score is the
    # largest of those left
    w["correction"] = torch.tensor([-5.0, -5.0, -5.0, -5.0, -5.0, -5.0, -5.0, -9.0], dtype=torch.float64)
    idx, _ = ps.route(h, {"router": {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}}, w)
    assert sorted(idx[0].tolist()) == [2, 3, 5]


def test_plain_feed_forwards():
    h = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    w = {"up": torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 0.5]], dtype=torch.float64),
         "down": torch.tensor([[1.0, 1.0, 1.0]], dtype=torch.float64)}
    assert float(ps.dense_ff(h, w)) == 1.0 + 0.0 + 1.0          # relu(1)^2 + relu(-2)^2 + relu(1)^2
    e = {"e0.gate": torch.tensor([[1.0, 0.0]], dtype=torch.float64), "e0.up": torch.tensor([[0.0, 1.0]], dtype=torch.float64),
         "e0.down": torch.tensor([[3.0]], dtype=torch.float64)}
    want = 3.0 * (1.0 / (1.0 + math.exp(-1.0))) * -2.0
    assert abs(float(ps.expert(h, e, "e0.")) - want) < 1e-12
    assert torch.allclose(ps.offset_norm(torch.tensor([[3.0, 4.0]], dtype=torch.float64), torch.tensor([0.0, 1.0], dtype=torch.float64), 0.0),
                          torch.tensor([[3.0, 8.0]], dtype=torch.float64) / math.sqrt(12.5))
