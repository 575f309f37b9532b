"""Matusun's configuration, builder and run order on the CPU, and the plain implementation's
mechanisms against special cases."""
import copy

import pytest
import torch

import plain_matusun as pm
from matusun_configs import MATUSUN, matusun


def test_config_reads_every_size_and_constant():
    from pytriton_llama_amd.config import MatusunConfig
    cfg, _, _ = matusun("M1")
    c = MatusunConfig.from_dict(cfg)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, len(c.layers), c.streams) == (200, 64, 1e-5, 4, 3)
    assert [l.kind for l in c.layers] == ["attention", "mamba1", "attention", "mamba1"]
    a, s = c.layers[0].mixer, c.layers[3].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.window, a.rot_dims, a.rot_base) == \
        (4, 2, 16, 24, 0.3, 20, 8, 10000.0)
    assert (s.inner, s.state, s.dt_rank, s.conv) == (72, 24, 5, 3)
    m = c.layers[0].mlp
    assert (m.ff, m.experts, m.identity, m.top, m.scale, m.shared_ff) == (40, 5, 2, 2, 1.5, 48)
    assert c.layers[2].mlp is None and c.layers[1].mlp.shared_ff == 0
    assert (c.loop.start, c.loop.stop, c.loop.times) == (1, 3, 2)
    assert [i for i, _ in c.run_order()] == [0, 1, 2, 1, 2, 3]
    assert c.to_dict() == cfg
    plain, _, _ = matusun("M2")
    p = MatusunConfig.from_dict(plain)
    assert p.streams is None and p.loop is None and [i for i, _ in p.run_order()] == [0, 1, 2, 3]
    assert (p.layers[1].mixer.window, p.layers[1].mixer.rot_dims) == (None, 0)


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][0].update(type="delta"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "lacks 'scale'"),
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "dims 18"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size must be positive"),
    (lambda c: c["layers"][1]["mixer"].update(conv=0), "conv must be positive"),
    (lambda c: c["layers"][1]["mixer"].pop("dt_rank"), "lacks 'dt_rank'"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "unknown feed-forward kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=8), "top 8 of 5 + 2"),
    (lambda c: c["layers"][0]["mlp"]["router"].pop("scale"), "lacks 'scale'"),
    (lambda c: c["loop"].update(stop=5), "does not fit"),
    (lambda c: c["loop"].update(times=0), "does not fit"),
    (lambda c: c.update(streams=17), "streams"),
    (lambda c: c.pop("norm"), "lacks 'norm'"),
    (lambda c: c.update(layers=[]), "empty"),
])
def test_config_errors_name_the_place(change, text):
    from pytriton_llama_amd.config import ConfigError, MatusunConfig
    cfg, _, _ = matusun("M1")
    change(cfg)
    with pytest.raises(ConfigError) as e:
        MatusunConfig.from_dict(cfg)
    assert text in str(e.value)


@pytest.mark.parametrize("name", sorted(MATUSUN))
def test_builder_wires_caches_and_names(name):
    import pytriton_llama_amd  # noqa: F401
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.parts import PagedSpec, StateSpec
    cfg, _, _ = matusun(name)
    model = build_model(cfg)
    order = pm.run_order(cfg)
    assert [c.block for c in model.schedule] == order
    # every run of a layer has a cache layer of its own, of the kind its mixer keeps
    assert [c.cache_layer for c in model.schedule] == list(range(len(order)))
    for call in model.schedule:
        layer = cfg["layers"][call.block]
        spec = model.cache_layers[call.cache_layer]
        if layer["type"] == "attention":
            assert isinstance(spec, PagedSpec)
            assert spec.window == (layer["mixer"].get("mask") or {}).get("size")
        else:
            m = layer["mixer"]
            assert isinstance(spec, StateSpec) and spec.dtype == torch.float32
            assert spec.shape == (m["inner"] * m["state"] + (m["conv"] - 1) * m["inner"],)
    names = set(model.expected_tensors())
    assert {"embed", "final.norm", "l0.norm1"} <= names and not any(n.startswith("head") for n in names)
    for i, layer in enumerate(cfg["layers"]):
        has_hc = "streams" in cfg
        assert (f"l{i}.hc1.mix" in names) == has_hc
        assert (f"l{i}.hc2.in" in names) == (has_hc and layer["mlp"] is not None)
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None)
        if layer["type"] == "attention":
            assert {f"l{i}.mix.q", f"l{i}.mix.q.norm", f"l{i}.mix.k.norm", f"l{i}.mix.o"} <= names
        else:
            assert {f"l{i}.mix.in", f"l{i}.mix.conv", f"l{i}.mix.conv.b", f"l{i}.mix.x", f"l{i}.mix.dt",
                    f"l{i}.mix.dt.b", f"l{i}.mix.A_log", f"l{i}.mix.D", f"l{i}.mix.o"} <= names
        if layer["mlp"] is not None:
            r = layer["mlp"]["router"]
            E = r["experts"]
            assert model.expected_tensors()[f"l{i}.mlp.router"][1].shape == (E + r.get("identity", 0), cfg["width"])
            assert f"l{i}.mlp.e{E - 1}.up" in names and f"l{i}.mlp.e{E}.up" not in names
            assert f"l{i}.mlp.e0.gate" not in names
            assert (f"l{i}.mlp.shared.up" in names) == ("shared" in layer["mlp"])


def test_groups_of_the_cache_manager():
    """Attention layers with equal sizes and windows share a page pool; every run of a scan has a
    state of its own in the request's slot."""
    import pytriton_llama_amd  # noqa: F401
    from pytriton_llama_amd.cache import CacheManager
    from pytriton_llama_amd.config import build_model
    cfg, _, page = matusun("M1")
    model = build_model(cfg)
    man = CacheManager(model.cache_layers, page, 32, 2)
    assert len(man.paged) == 1 and len(man.paged[0].layers) == 3        # layer 0 once, layer 2 twice
    assert sorted(len(g.layers) for g in man.states) == [1, 2]          # layer 3 once, layer 1 twice


# ---- the plain implementation against special cases --------------------------------------------
def test_plain_window_and_rotation():
    vis = pm.window_mask(6, 3)
    assert vis[5].tolist() == [False, False, False, True, True, True] and vis[1].tolist()[:3] == [True, True, False]
    assert pm.window_mask(4, None).sum() == 10
    x = torch.randn(5, 2, 8, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 1000])
    y = pm.rotate_half(x, pos, 4, 100.0)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    assert torch.allclose(y[..., :4].norm(dim=-1), x[..., :4].norm(dim=-1))
    # a rotation: the product of a rotated query and key depends on the distance alone
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    a = (pm.rotate_half(q, torch.tensor([7]), 8, 50.0) * pm.rotate_half(k, torch.tensor([3]), 8, 50.0)).sum()
    b = (pm.rotate_half(q, torch.tensor([104]), 8, 50.0) * pm.rotate_half(k, torch.tensor([100]), 8, 50.0)).sum()
    assert abs(float(a - b)) < 1e-9


def test_plain_scan_is_a_decaying_sum():
    """With one state, B = C = 1 and a constant step the scan is a geometric sum of the inputs."""
    T = 6
    x = torch.randn(T, 1, dtype=torch.float64)
    dt = torch.full((T, 1), 0.5, dtype=torch.float64)
    A = torch.tensor([[-2.0]], dtype=torch.float64)
    ones = torch.ones(T, 1, dtype=torch.float64)
    y = pm.selective_scan(x, dt, A, ones, ones, torch.tensor([3.0], dtype=torch.float64))
    decay = float(torch.exp(torch.tensor(-1.0, dtype=torch.float64)))
    for t in range(T):
        want = sum(0.5 * float(x[s]) * decay ** (t - s) for s in range(t + 1)) + 3.0 * float(x[t])
        assert abs(float(y[t]) - want) < 1e-12
    c = pm.causal_conv(torch.arange(1.0, 5.0, dtype=torch.float64)[:, None], torch.tensor([[1.0, 10.0, 100.0]],
                       dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64))
    assert c[:, 0].tolist() == [100.5, 210.5, 321.5, 432.5]


def test_plain_router():
    h = torch.eye(4, dtype=torch.float64)
    router = torch.tensor([[5.0, 0, 0, 0], [0, 5.0, 0, 0], [4.0, 4.0, 0, 0]], dtype=torch.float64)
    corr = torch.tensor([0.0, 0.0, 10.0], dtype=torch.float64)
    idx, wgt, s = pm.route(h, router, corr, 2, 2.0)
    assert torch.allclose(s.sum(-1), torch.ones(4, dtype=torch.float64))
    assert all(2 in row for row in idx.tolist())            # the correction puts output 2 first everywhere
    assert torch.allclose(wgt.sum(-1), torch.full((4,), 2.0, dtype=torch.float64))
    assert idx[0].tolist() == [2, 0] and abs(float(wgt[0, 0] / wgt[0, 1]) - float(s[0, 2] / s[0, 0])) < 1e-12
    # an expert that returns its input: with one real expert of zeros the layer is weight * h
    mlp = {"router": {"experts": 1, "identity": 2, "top": 1, "scale": 1.5}}
    w = {"router": torch.tensor([[0.0] * 4, [0.0] * 4, [9.0] * 4], dtype=torch.float64),
         "correction": torch.zeros(3, dtype=torch.float64),
         "e0.up": torch.zeros(3, 4, dtype=torch.float64), "e0.down": torch.zeros(4, 3, dtype=torch.float64)}
    x = torch.randn(5, 4, dtype=torch.float64).abs() + 1
    assert torch.allclose(pm.routed_mlp(x, mlp, w), 1.5 * x)


def test_plain_streams():
    """One stream with coefficients of one is the plain residual sum; the loop repeats layers."""
    T, W = 3, 4
    x = torch.randn(1, T, W, dtype=torch.float64)
    hc = {"in": torch.ones(1, dtype=torch.float64), "mix": torch.ones(1, 1, dtype=torch.float64),
          "out": torch.ones(1, dtype=torch.float64)}
    nw = torch.ones(W, dtype=torch.float64)
    y = pm.hyper_sublayer(x, hc, nw, 1e-6, lambda a: 2 * a)
    assert torch.allclose(y[0], x[0] + 2 * pm.rms(x[0], 1e-6))
    assert pm.run_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert pm.run_order({"layers": [0] * 2}) == [0, 1]
